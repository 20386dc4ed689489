"""GPU parity of the Dion path against the CPU oracle (reference dion/dion.py:742-875), through the C ABI."""
import pytest
import torch

from conftest import rel_fro

pytestmark = pytest.mark.gpu

ORTH_TOL = 1e-3   # ||P^T P - I||_F (north star)
FP32_TOL = 1e-4   # M, Q (sign-aligned), X relative error in the all-fp32 configuration


def _sign_align(a, ref):
    """Flip columns of `a` to agree in sign with `ref` (thin-QR factors are unique up to column signs)."""
    s = torch.sign((a.double() * ref.double()).sum(dim=0))
    s[s == 0] = 1
    return a.double() * s


@pytest.mark.parametrize("rows,r", [(768, 192), (3072, 768), (768, 768), (520, 72), (4096, 512), (100, 28), (100, 27)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_orthonormalize(dev, rows, r, dtype):
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(0)
    # a badly conditioned factor: Gaussian times a graded diagonal (cond ~ 1e4)
    P = torch.randn(rows, r, dtype=torch.float64) * torch.logspace(0, -4, r, dtype=torch.float64)
    P = P.to(dtype)
    Q, info = orthonormalize(P.to(dev), return_info=True)
    assert Q.dtype == dtype and Q.shape == P.shape and int(info.item()) == 0
    Qd = Q.double().cpu()
    orth = (Qd.T @ Qd - torch.eye(r, dtype=torch.float64)).norm().item()
    print(f"orth {rows}x{r} {dtype}: ||QtQ-I|| = {orth:.2e}")
    assert orth <= (ORTH_TOL if dtype == torch.float32 else 5e-2 * (r ** 0.5) / 8)  # bf16 storage of Q: ~2^-9 per entry
    # same factor as Householder QR of the same (rounded) input, up to column signs, and R upper triangular
    Qh, Rh = torch.linalg.qr(P.double())
    if dtype == torch.float32:
        assert rel_fro(_sign_align(Qd, Qh), Qh) <= 2e-3   # conditioning-limited: cond(P) * eps32 ~ 1e-3
    Rm = Qd.T @ P.double()
    assert (Rm.tril(-1).norm() / Rm.norm()).item() <= (1e-5 if dtype == torch.float32 else 2e-2)
    assert (torch.diagonal(Rm) > 0).all()


@pytest.mark.parametrize("rows,r", [(768, 192), (2048, 320), (1024, 64)])
def test_ragged_rank_products_same_bits_on_either_k_loop(dev, rows, r):
    """The bf16 products of a rank that is not a whole number of tiles run the direct-to-LDS K loop with edge tiles;
    the bounds-checked K loop (option "edge_loop" = 0) gives the same bits -- including the stacked product
    `[P P] [T_hi; T_lo]`, whose A operand is read twice along k."""
    from dion_amd import _lib
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(3)
    P = (torch.randn(2, rows, r, dtype=torch.float64) * torch.logspace(0, -2, r, dtype=torch.float64)).to(torch.bfloat16).to(dev)
    try:
        _lib.set_option("edge_loop", 1)
        Q1, i1 = orthonormalize(P.clone(), return_info=True)
        _lib.set_option("edge_loop", 0)
        Q0, i0 = orthonormalize(P.clone(), return_info=True)
    finally:
        _lib.set_option("edge_loop", -1)
    assert bool((i1 == 0).all()) and bool((i0 == 0).all())
    assert torch.equal(Q1, Q0)


@pytest.mark.parametrize("rows,r,batch", [(1536, 200, 3), (1024, 72, 2), (2048, 192, 4), (3072, 520, 1),
                                          (16384, 256, 1), (12296, 136, 2)])
def test_orthonormalize_bf16_ragged_ranks(dev, rows, r, batch):
    """bf16 factors with `rows >= 4 r` take the fp32 pass on the bf16 matrix cores; ranks that are not multiples
    of 64 leave a ragged last block column in the blocked Cholesky and in the rows of the inverse factor.  The
    result must be orthonormal to bf16 rounding and span what Householder QR of the same matrix spans.
    The last two cases are tall and narrow: their Gram products run as 16 and 22 K slices (the last one ragged) and
    the finishing pass splits the column blocks across workgroups."""
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(11)
    P = torch.randn(batch, rows, r).bfloat16()
    Q, info = orthonormalize(P.to(dev), return_info=True)
    assert Q.dtype == torch.bfloat16 and (info == 0).all()
    Qd = Q.double().cpu()
    eye = torch.eye(r, dtype=torch.float64)
    for b in range(batch):
        orth = (Qd[b].T @ Qd[b] - eye).norm().item()
        Qh, _ = torch.linalg.qr(P[b].double())
        # projector onto the span, compared with Householder's (column signs and bf16 rounding aside)
        span = ((Qd[b] @ (Qd[b].T @ Qh)) - Qh).norm().item() / Qh.norm().item()
        diff = rel_fro(_sign_align(Qd[b], Qh), Qh)
        print(f"{rows}x{r} matrix {b}: ||QtQ-I|| = {orth:.2e}, span defect {span:.2e}, vs Householder {diff:.2e}")
        assert orth <= 3e-2 * (r / 200) ** 0.5 and span <= 5e-3 and diff <= 5e-3


@pytest.mark.parametrize("log_cond,passes,tol", [(4, 1, 5e-6), (6, 2, 5e-5), (7, 2, 2e-4), (7.5, 3, 5e-5)])
def test_orthonormalize_conditioning(dev, log_cond, passes, tol):
    """Genuinely ill-conditioned factors (singular values graded over `log_cond` decades between random
    orthonormal bases, not a column scaling that a Cholesky factorisation does not feel).  The fp64 pass
    leaves ||Q^T Q - I|| ~ eps64 * cond^2 and every fp32 polishing pass squares what is left, down to fp32
    round-off; the optimizer runs two passes, so it holds the 1e-3 bar up to cond ~ 2e7."""
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(5)
    rows, r = 1536, 320
    U, _ = torch.linalg.qr(torch.randn(rows, r, dtype=torch.float64))
    V, _ = torch.linalg.qr(torch.randn(r, r, dtype=torch.float64))
    P = ((U * torch.logspace(0, -log_cond, r, dtype=torch.float64)) @ V.T).float()
    Q, info = orthonormalize(P.to(dev), passes=passes, return_info=True)
    assert int(info.item()) == 0
    Qd = Q.double().cpu()
    orth = (Qd.T @ Qd - torch.eye(r, dtype=torch.float64)).norm().item()
    Qh, _ = torch.linalg.qr(P.double())
    diff = rel_fro(_sign_align(Qd, Qh), Qh)
    print(f"cond 1e{log_cond}, {passes} passes: ||QtQ-I|| = {orth:.2e}, vs Householder {diff:.2e}")
    assert orth <= tol and diff <= tol


def test_orthonormalize_batch_and_rank_deficient(dev):
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(1)
    P = torch.randn(3, 512, 128)
    P[1, :, 40] = 0.0                      # a zero column: pivot 0 at column 40
    P[2] = 0.0                             # an all-zero matrix
    Q, info = orthonormalize(P.to(dev), return_info=True)
    info = info.cpu().tolist()
    assert info[0] == 0 and info[1] == 41 and info[2] == 1
    assert torch.isfinite(Q).all()
    Q0 = Q[0].double().cpu()
    assert (Q0.T @ Q0 - torch.eye(128, dtype=torch.float64)).norm().item() <= ORTH_TOL
    assert torch.count_nonzero(Q[2]) == 0 and torch.count_nonzero(Q[1][:, 40]) == 0
    # batch independence
    assert torch.equal(orthonormalize(P[0].to(dev)), Q[0])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_orthonormalize_numerically_rank_deficient(dev, dtype):
    """P = A B of rank 96 < r = 128: the dependent columns have pivots at round-off level of either sign.  They must
    not come back as scaled noise: the result is finite, every column is a unit vector or zero, the kept columns
    are orthonormal, and `info` reports the first dropped column."""
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(3)
    rows, r, k = 1024, 128, 96
    P = (torch.randn(rows, k, dtype=torch.float64) @ torch.randn(k, r, dtype=torch.float64)).to(dtype)
    Q, info = orthonormalize(P.to(dev), return_info=True)
    assert torch.isfinite(Q).all()
    Qd = Q.double().cpu()
    norms = Qd.norm(dim=0)
    kept = norms > 0.5
    tol = 1e-3 if dtype == torch.float32 else 3e-2
    assert ((norms[kept] - 1).abs() <= tol).all() and (norms[~kept] == 0).all()
    if dtype == torch.float32:
        assert int(info.item()) != 0
        assert int(kept.sum()) >= k - 2 and int(kept.sum()) <= k + 2
    else:
        # rounded to bf16 the dependent columns carry 2^-9 of independent noise: P has full rank with a condition
        # number of a few thousand, and keeping every column is as valid as dropping the noisy ones
        assert (int(info.item()) != 0) == (int(kept.sum()) < r)
    Qk = Qd[:, kept]
    assert (Qk.T @ Qk - torch.eye(Qk.shape[1], dtype=torch.float64)).norm().item() <= (ORTH_TOL if dtype == torch.float32 else 0.3)
    # the kept columns span P's column space
    resid = P.double() - Qk @ (Qk.T @ P.double())
    assert (resid.norm() / P.double().norm()).item() <= (1e-4 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,r", [(768, 192), (3072, 512)])
def test_orthonormalize_fp32_first_pass_agrees_with_the_fp64_pass(dev, dtype, rows, r):
    """A well-conditioned factor takes the fp32 pass (two passes asked for, rows >= 4 r); three passes always run the
    fp64 pass.  Same thin-QR factor either way."""
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(4)
    P = torch.randn(4, rows, r).to(dtype).to(dev)
    Qa, ia = orthonormalize(P, passes=2, return_info=True)
    Qb, ib = orthonormalize(P, passes=3, return_info=True)
    assert ia.abs().sum().item() == 0 and ib.abs().sum().item() == 0
    d = rel_fro(Qa.double().cpu(), Qb.double().cpu())
    print(f"fp32-first vs fp64 pass, {rows}x{r} {dtype}: {d:.2e}")
    assert d <= (2e-5 if dtype == torch.float32 else 4e-3)
    Qd = Qa[0].double().cpu()
    orth = (Qd.T @ Qd - torch.eye(r, dtype=torch.float64)).norm().item()
    assert orth <= (2e-5 if dtype == torch.float32 else 5e-2 * (r ** 0.5) / 8)


def test_dion_step_with_a_rank_deficient_gradient_stays_bounded(dev):
    """First step from zero momentum with a gradient of rank 8 < r = 64: B Q has rank 8."""
    from dion_amd import Dion

    torch.manual_seed(6)
    m, n = 512, 256
    p = torch.nn.Parameter((torch.randn(m, n) * 0.02).to(dev))
    opt = Dion([p], rank_fraction=0.25, lr=0.01, mu=0.95, weight_decay=0.0)
    x0 = p.detach().clone()
    for _ in range(3):
        p.grad = ((torch.randn(m, 8) @ torch.randn(8, n)) * 1e-3).to(dev)
        opt.step()
    torch.cuda.synchronize()
    st = opt.state[p]
    assert torch.isfinite(p).all() and torch.isfinite(st["momentum"]).all() and torch.isfinite(st["Q"]).all()
    # an orthonormal P bounds the update: ||P Qn^T||_F <= sqrt(r), scaled by lr * sqrt(m / n)
    step_bound = 0.01 * (m / n) ** 0.5 * (64 ** 0.5) * 1.05
    assert (p.detach() - x0).norm().item() <= 3 * step_bound
    assert st["momentum"].norm().item() <= 3 * (1e-3 * 8 ** 0.5 * (m * n) ** 0.5) * 1.5


def _run_dion(dev, shapes, rank_fraction, steps, x_dtype, m_dtype, q_dtype, seed_q=2, seed_g=3, lr=0.01, mu=0.95, wd=0.01,
              check=None):
    from dion_amd import Dion, DionMixedPrecisionConfig
    from oracle import dion_step as O

    g0 = torch.Generator().manual_seed(11)
    X0 = [(torch.randn(s, generator=g0) * 0.02).to(x_dtype) for s in shapes]
    gq = torch.Generator().manual_seed(seed_q)
    Q0 = []
    for (m, n) in shapes:
        r = O.rank_of(m, n, rank_fraction)
        q = torch.randn((m if m < n else n, r), generator=gq)
        Q0.append((q / q.norm(dim=0, keepdim=True)).to(q_dtype))
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    opt = Dion(params, rank_fraction=rank_fraction, lr=lr, mu=mu, weight_decay=wd,
               mixed_precision_config=DionMixedPrecisionConfig(momentum_dtype=m_dtype, Q_dtype=q_dtype))
    Xo = [x.clone() for x in X0]
    Mo = [torch.zeros_like(x, dtype=m_dtype) for x in X0]
    Qo = [q.clone() for q in Q0]
    gg = torch.Generator().manual_seed(seed_g)
    sk = torch.Generator().manual_seed(0)
    for step in range(steps):
        G = [(torch.randn(s, generator=gg) * 1e-3).to(x_dtype) for s in shapes]
        for p, g in zip(params, G):
            p.grad = g.to(dev)
        if step == 0:
            # lazily create the states, then inject the seeded Q (the reference draws it from the global RNG)
            for p, q in zip(params, Q0):
                st = opt._get_or_initialize_state(p, opt.param_groups[0])
                assert st["Q"].shape == q.shape and st["Q"].dtype == q_dtype and st["momentum"].dtype == m_dtype
                st["Q"].copy_(q.to(dev))
        O.dion_step(Xo, G, Mo, Qo, lr=lr, mu=mu, weight_decay=wd, generator=sk)
        opt.step()
        torch.cuda.synchronize()
        check(step, params, opt, Xo, Mo, Qo)
    return opt


@pytest.mark.parametrize("shapes,rank_fraction", [
    ([(768, 768), (3072, 768), (768, 3072)], 0.25),
    ([(512, 1024), (1024, 512), (256, 256)], 0.5),
])
def test_dion_fp32_matches_oracle_10_steps(dev, shapes, rank_fraction):
    """GPT-small Dion configuration (low rank) in all-fp32 state: M, Q (sign-aligned), X within 1e-4 after every step."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            eM = rel_fro(st["momentum"], Mo[i])
            eX = rel_fro(p.detach(), Xo[i])
            eQ = rel_fro(_sign_align(st["Q"].cpu(), Qo[i]), Qo[i])
            qn = st["Q"].double().norm(dim=0)
            assert eM <= FP32_TOL and eX <= FP32_TOL and eQ <= FP32_TOL, (step, i, eM, eX, eQ)
            assert (qn - 1).abs().max().item() < 1e-5
        info = torch.cat([v for v in opt.cholesky_info().values()])
        assert int(info.abs().sum().item()) == 0

    _run_dion(dev, shapes, rank_fraction, 10, torch.float32, torch.float32, torch.float32, check=check)


@pytest.mark.parametrize("shapes,rank_fraction", [
    ([(768, 768), (1536, 768), (768, 1536)], 0.3),      # r = 231: aligned matrices, rank off the 8-grid
    ([(100, 60), (60, 100), (50, 50), (101, 100)], 0.45),  # r = 27 / 27 / 23 / 45: nothing on the grid
])
def test_dion_shapes_and_ranks_off_the_alignment_grid(dev, shapes, rank_fraction):
    """Ranks that are not multiples of 8 run with zero columns up to the next multiple inside the library, other
    matrix dimensions on zero-padded copies made by the host side: same 1e-4 bar as any other shape."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            assert st["Q"].shape == Qo[i].shape and st["momentum"].shape == p.shape
            eM = rel_fro(st["momentum"], Mo[i])
            eX = rel_fro(p.detach(), Xo[i])
            eQ = rel_fro(_sign_align(st["Q"].cpu(), Qo[i]), Qo[i])
            assert eM <= FP32_TOL and eX <= FP32_TOL and eQ <= FP32_TOL, (step, i, eM, eX, eQ)
        info = torch.cat([v for v in opt.cholesky_info().values()])
        assert int(info.abs().sum().item()) == 0

    _run_dion(dev, shapes, rank_fraction, 5, torch.float32, torch.float32, torch.float32, check=check)


def test_dion_bf16_off_the_alignment_grid(dev):
    """The bf16 configuration (bf16 weights and momentum, fp32 Q) at a rank and at dimensions off the 8-grid."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            assert eM <= 1e-2 and eX <= 1e-2, (step, i, eM, eX)
            assert (st["Q"].double().norm(dim=0) - 1).abs().max().item() < 1e-2

    _run_dion(dev, [(768, 768), (300, 100), (100, 300)], 0.3, 5, torch.bfloat16, torch.bfloat16, torch.float32,
              check=check)


def test_dion_bucket_larger_than_one_chunk(dev):
    """70 same-shape matrices: more than the 64 a launch's pointer tables hold, so the bucket goes through the
    library in two chunks (status words and pointer tables at an offset)."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            eQ = rel_fro(_sign_align(st["Q"].cpu(), Qo[i]), Qo[i])
            assert eM <= FP32_TOL and eX <= FP32_TOL and eQ <= FP32_TOL, (step, i, eM, eX, eQ)
        info = torch.cat([v for v in opt.cholesky_info().values()])
        assert info.numel() == 70 and int(info.abs().sum().item()) == 0

    _run_dion(dev, [(64, 48)] * 70, 0.5, 2, torch.float32, torch.float32, torch.float32, check=check)


def test_dion_fp32_full_rank(dev):
    """rank_fraction 1.0: square matrices are conditioning-limited (cond(BQ) ~ 1e5-1e6): the reference's own
    fp32-vs-fp64 spread in Q is ~7e-4 there, while M and X stay tight.  At full rank M_new = mu * B exactly."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            eQ = rel_fro(_sign_align(st["Q"].cpu(), Qo[i]), Qo[i])
            print(f"full rank step {step} matrix {i}: M {eM:.2e} X {eX:.2e} Q {eQ:.2e}")
            assert eM <= FP32_TOL and eX <= FP32_TOL
            assert eQ <= (5e-3 if p.shape[0] == p.shape[1] else FP32_TOL * 3)

    _run_dion(dev, [(768, 768), (1536, 768), (768, 1536)], 1.0, 4, torch.float32, torch.float32, torch.float32, check=check)


def test_dion_bf16_momentum(dev):
    """Storage of the bf16 Dion configurations: bf16 weights and momentum, fp32 Q.  Every product rounds to bf16, so the
    bar is bf16-level (1e-2) on M and X; P's invariants are checked on the GPU result itself."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            assert st["momentum"].dtype == torch.bfloat16 and st["Q"].dtype == torch.float32
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            assert eM <= 1e-2 and eX <= 1e-2, (step, i, eM, eX)
            qn = st["Q"].double().norm(dim=0)
            assert (qn - 1).abs().max().item() < 1e-2

    _run_dion(dev, [(768, 768), (3072, 768), (768, 3072)], 0.25, 10, torch.bfloat16, torch.bfloat16, torch.float32,
              check=check)


def test_dion_fp32_momentum_with_bf16_weights(dev):
    """`DionMixedPrecisionConfig(momentum_dtype=float32)` on bf16 parameters (the reference accepts it:
    `foreach_baddbmm_` adds the fp32 update into the bf16 weights, dion/dion.py:1513-1530): fp32 factors, bf16 X."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            assert p.dtype == torch.bfloat16 and st["momentum"].dtype == torch.float32
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            eQ = rel_fro(_sign_align(st["Q"].cpu(), Qo[i]), Qo[i])
            assert eM <= FP32_TOL and eQ <= FP32_TOL, (step, i, eM, eQ)
            # bf16 weights: the two runs may round an element differently once in a while
            assert eX <= 2e-3, (step, i, eX)
            assert (p.detach().cpu() == Xo[i]).float().mean().item() > 0.98

    _run_dion(dev, [(256, 128), (128, 256), (192, 192)], 0.25, 4, torch.bfloat16, torch.float32, torch.float32,
              check=check)


def test_dion_all_zero_gradient(dev):
    """All-zero B: P = 0, Q_new = colnorm(Q), M = 0, X = (1 - lr wd) X (reference dion/dion.py:1416-1444)."""
    from dion_amd import Dion

    torch.manual_seed(0)
    p = torch.nn.Parameter(torch.randn(256, 128, device=dev))
    x0 = p.detach().clone()
    p.grad = torch.zeros_like(p)
    opt = Dion([p], rank_fraction=0.5, lr=0.01, weight_decay=0.1)
    st = opt._get_or_initialize_state(p, opt.param_groups[0])
    q0 = st["Q"].clone()
    opt.step()
    assert torch.count_nonzero(st["momentum"]) == 0
    assert torch.allclose(p.detach(), x0 * (1 - torch.tensor(0.01) * torch.tensor(0.1)).item(), rtol=1e-6, atol=0)
    assert torch.allclose(st["Q"], q0 / (q0.norm(dim=0, keepdim=True) + 1e-8), rtol=1e-5, atol=1e-7)
    assert torch.isfinite(st["Q"]).all()


def test_dion_groups_and_validation(dev):
    from dion_amd import Dion

    w = torch.nn.Parameter(torch.randn(128, 64, device=dev))
    b = torch.nn.Parameter(torch.zeros(64, device=dev))
    opt = Dion([dict(params=[w], rank_fraction=0.25, rank_multiple_of=8), dict(params=[b], algorithm="lion")], lr=0.01)
    w.grad, b.grad = torch.randn_like(w), torch.ones_like(b)
    opt.step()
    assert opt.state[w]["Q"].shape == (64, 16) and set(opt.state[w]) == {"momentum", "Q"}
    assert torch.allclose(b.detach(), torch.full_like(b, -0.01))
    sd = opt.state_dict()
    assert sd["param_groups"][0]["step"] == 1 and sd["param_groups"][0]["algorithm"] == "dion"
    opt2 = Dion([dict(params=[w], rank_fraction=0.25, rank_multiple_of=8), dict(params=[b], algorithm="lion")], lr=0.01)
    opt2.load_state_dict(sd)
    assert torch.equal(opt2.state[w]["Q"], opt.state[w]["Q"])
    t3 = torch.nn.Parameter(torch.randn(4, 8, 8, device=dev))
    t3.grad = torch.randn_like(t3)
    with pytest.raises(NotImplementedError):
        Dion([t3]).step()


@pytest.mark.parametrize("qr_method,power_iters", [("cqr", 1), ("qr", 2), ("rcqr", 3)])
def test_dion_reference_class(dev, qr_method, power_iters):
    """`DionReference` (reference dion/dion_reference.py:64-365): every `qr_method` name and several power
    iterations against the oracle's per-matrix update, all-fp32 state, 1e-4 on M, X and sign-aligned Q."""
    from dion_amd import DionMixedPrecisionConfig, DionReference
    from oracle import dion_step as O

    shapes = [(512, 256), (256, 512), (200, 120)]
    rank_fraction = 0.25
    g = torch.Generator().manual_seed(31)
    X0 = [torch.randn(s, generator=g) * 0.02 for s in shapes]
    Q0 = []
    for (m, n) in shapes:
        q = torch.randn((m if m < n else n, O.rank_of(m, n, rank_fraction)), generator=g)
        Q0.append(q / q.norm(dim=0, keepdim=True))
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    cfg = DionMixedPrecisionConfig(momentum_dtype=torch.float32, Q_dtype=torch.float32)
    opt = DionReference(params, rank_fraction=rank_fraction, lr=0.01, mu=0.95, weight_decay=0.01, qr_method=qr_method,
                        power_iters=power_iters, cqr_warmup_steps=1, mixed_precision_config=cfg)
    Xo, Mo, Qo = [x.clone() for x in X0], [torch.zeros_like(x) for x in X0], [q.clone() for q in Q0]
    sk = torch.Generator().manual_seed(0)
    for step in range(4):
        G = [torch.randn(s, generator=g) * 1e-3 for s in shapes]
        for p, gr in zip(params, G):
            p.grad = gr.to(dev)
        if step == 0:
            for p, q in zip(params, Q0):
                opt._get_or_initialize_state(p, opt.param_groups[0])["Q"].copy_(q.to(dev))
        for i in range(len(shapes)):
            Qo[i] = O.dion_update_reference(Xo[i], G[i], Mo[i], Qo[i], 0.01, 0.95, 0.01, 1e-8, power_iters=power_iters,
                                            qr_method=qr_method, generator=sk)
        opt.step()
        for i, p in enumerate(params):
            st = opt.state[p]
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            eQ = rel_fro(_sign_align(st["Q"].cpu(), Qo[i]), Qo[i])
            assert eM <= FP32_TOL and eX <= FP32_TOL and eQ <= FP32_TOL, (step, i, eM, eX, eQ)
    with pytest.raises(ValueError):
        DionReference(params, power_iters=0)
    with pytest.raises(ValueError):
        DionReference(params, qr_method="svd")


def test_orthonormalize_methods(dev):
    """The three `qr_method`s of the per-matrix reference class (dion/dion_reference.py:733-789) on the device: "cqr" is
    one CholeskyQR pass in fp32 and leaves a defect of about eps32 * cond(P)^2 (as the reference's does); "rcqr" and
    "qr" are orthonormal to round-off; all three are the same thin-QR factor."""
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(8)
    rows, r = 2048, 256
    U, _ = torch.linalg.qr(torch.randn(rows, r, dtype=torch.float64))
    V, _ = torch.linalg.qr(torch.randn(r, r, dtype=torch.float64))
    P = ((U * torch.logspace(0, -2.5, r, dtype=torch.float64)) @ V.T).float()     # cond ~ 300
    Qh, _ = torch.linalg.qr(P.double())
    eye = torch.eye(r, dtype=torch.float64)
    res = {}
    for method in ("rcqr", "qr", "cqr"):
        Q, info = orthonormalize(P.to(dev), qr_method=method, return_info=True)
        assert int(info.item()) == 0
        Qd = Q.double().cpu()
        res[method] = ((Qd.T @ Qd - eye).norm().item(), rel_fro(_sign_align(Qd, Qh), Qh))
        print(f"{method}: ||QtQ-I|| = {res[method][0]:.2e}, vs Householder {res[method][1]:.2e}")
    assert res["rcqr"][0] <= 2e-5 and res["qr"][0] <= 2e-5
    assert 1e-5 <= res["cqr"][0] <= 5e-2          # eps32 * cond^2 ~ 5e-3: visibly a single fp32 pass
    assert res["rcqr"][1] <= 5e-4 and res["qr"][1] <= 1e-5 and res["cqr"][1] <= 5e-2
    # "cqr" on a factor whose Cholesky factorisation fails: the fall-back runs on the device and reports the column
    Pz = torch.randn(2, 512, 64)
    Pz[1, :, 17] = 0.0
    Q, info = orthonormalize(Pz.to(dev), qr_method="cqr", return_info=True)
    assert info.cpu().tolist() == [0, 18] and torch.isfinite(Q).all() and torch.count_nonzero(Q[1][:, 17]) == 0
    Q1 = Q[1].double().cpu()
    keep = [j for j in range(64) if j != 17]
    assert (Q1[:, keep].T @ Q1[:, keep] - torch.eye(63, dtype=torch.float64)).norm().item() <= ORTH_TOL


@pytest.mark.parametrize("rows,r", [(100, 24), (1004, 64), (1001, 16)])
@pytest.mark.parametrize("method", ["rcqr", "qr", "cqr"])
def test_orthonormalize_bf16_with_rows_off_the_8_grid(dev, rows, r, method):
    """A bf16 factor whose rank is a multiple of 8 but whose number of rows is not: the Gram products on the bf16
    matrix cores sum over the rows in 16-byte chunks and do not apply; the fp32 kernels take such a factor (the entry
    point only asks for rows >= r).  All three methods must return the thin-QR factor."""
    from dion_amd.newton_schulz import orthonormalize

    torch.manual_seed(13)
    P = torch.randn(2, rows, r).bfloat16()
    Q, info = orthonormalize(P.to(dev), qr_method=method, return_info=True)
    assert Q.dtype == torch.bfloat16 and (info == 0).all()
    for b in range(2):
        Qd = Q[b].double().cpu()
        orth = (Qd.T @ Qd - torch.eye(r, dtype=torch.float64)).norm().item()
        Qh, _ = torch.linalg.qr(P[b].double())
        diff = rel_fro(_sign_align(Qd, Qh), Qh)
        print(f"{method} {rows}x{r} matrix {b}: ||QtQ-I|| = {orth:.2e}, vs Householder {diff:.2e}")
        assert orth <= 3e-2 and diff <= 5e-3


@pytest.mark.parametrize("dtype,rows,r,batch", [(torch.float32, 768, 192, 2), (torch.float32, 520, 72, 3),
                                                (torch.bfloat16, 3072, 192, 2), (torch.bfloat16, 1024, 64, 1)])
def test_orthonormalize_with_an_injected_sketch(dev, dtype, rows, r, batch):
    """The reference's randomised Cholesky QR with the sketch given by the caller (dion/dion.py:1287-1303,
    `generate_random_sketch_matrix` 1221-1263) against `oracle.orthogonalize` on the SAME sketch, up to column signs;
    the sketch only preconditions, so the sketch-free orthonormaliser must agree as well."""
    from dion_amd.dion import generate_random_sketch_matrix
    from dion_amd.newton_schulz import orthonormalize
    from oracle import dion_step as O

    torch.manual_seed(17)
    P = (torch.randn(batch, rows, r, dtype=torch.float64) * torch.logspace(0, -2, r, dtype=torch.float64)).to(dtype)
    Pd = P.to(dev)
    S = generate_random_sketch_matrix(Pd, 1.25, generator=torch.Generator(device=dev).manual_seed(3))
    k = 128 * -(-int(1.25 * r) // 128)
    assert S.shape == (batch, k, rows) and S.dtype == dtype and S.is_cuda
    assert abs(S.float().std().item() - (1.0 / k) ** 0.5) <= 0.05 * (1.0 / k) ** 0.5
    Q, info = orthonormalize(Pd, sketch=S, return_info=True)
    assert Q.dtype == dtype and (info == 0).all()
    ref = O.orthogonalize(P, sketch=S.cpu())
    plain = orthonormalize(Pd)
    tol = 2e-5 if dtype == torch.float32 else 8e-3
    for b in range(batch):
        Qd = Q[b].double().cpu()
        e_ref = rel_fro(_sign_align(Qd, ref[b]), ref[b])
        e_plain = rel_fro(_sign_align(plain[b].double().cpu(), Qd), Qd)
        orth = (Qd.T @ Qd - torch.eye(r, dtype=torch.float64)).norm().item()
        print(f"sketched {dtype} {rows}x{r} matrix {b}: vs oracle {e_ref:.2e}, vs sketch-free {e_plain:.2e}, ||QtQ-I|| {orth:.2e}")
        assert e_ref <= tol and e_plain <= tol
        assert orth <= (ORTH_TOL if dtype == torch.float32 else 5e-2 * (r ** 0.5) / 8)
    with pytest.raises(ValueError):
        orthonormalize(Pd, sketch=S, qr_method="cqr")
