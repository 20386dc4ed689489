"""The benchmark configurations at their full sizes under a checker: the CPU oracle on the same seeded inputs where
it finishes in seconds, through the public optimizer classes (which call the C ABI).

  config 2  full Muon step, GPT-small: 72 bf16 matrices, Nesterov                (reference dion/muon.py:356-486)
  config 3  full Dion step, GPT-small matrices, rank fraction 1.0, 10 steps      (reference dion/dion.py:742-875)
  config 4  one Llama-3-8B layer under Muon: 4096^2, 1024x4096, 14336x4096, 4096x14336
  config 5  Llama-3-70B MLP matrices under Dion, r = 512, 5 steps
"""
import pytest
import torch

from conftest import rel_fro
from test_gpu_dion import _run_dion, _sign_align

pytestmark = pytest.mark.gpu

GPT_SMALL_LAYER = [(768, 768)] * 4 + [(3072, 768), (768, 3072)]
LLAMA8B_LAYER = [(4096, 4096)] * 2 + [(1024, 4096)] * 2 + [(14336, 4096)] * 2 + [(4096, 14336)]


def test_config2_full_gpt_small_muon_step(dev):
    """All 72 matrices in one `Muon.step()`: the real 48 / 12 / 12 grouped launches.  Momentum bit exact, weights within
    the Newton-Schulz bar (2e-2 of the update) plus one bf16 rounding of the weight."""
    from dion_amd import Muon
    from oracle import muon_step as O

    shapes = GPT_SMALL_LAYER * 12
    gen = torch.Generator().manual_seed(1)
    X0 = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
    Xo, Mo = [x.clone() for x in X0], [torch.zeros_like(x) for x in X0]
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    lr, mu, wd = 0.02, 0.95, 0.01
    opt = Muon(params, lr=lr, mu=mu, weight_decay=wd, nesterov=True, adjust_lr="spectral_norm")
    decay = (1 - torch.tensor(lr) * torch.tensor(wd)).item()
    for step in range(2):
        G = [(torch.randn(s, generator=gen) * 1e-3).bfloat16() for s in shapes]
        for p, g in zip(params, G):
            p.grad = g.to(dev)
        prev = [x.clone() for x in Xo]
        O.muon_step(Xo, G, Mo, lr=lr, mu=mu, weight_decay=wd, epsilon=1e-8, nesterov=True)
        opt.step()
        torch.cuda.synchronize()
        worst = 0.0
        for i, p in enumerate(params):
            assert torch.equal(opt.state[p]["momentum"].cpu(), Mo[i]), f"momentum differs, matrix {i} step {step}"
            upd_ref = prev[i].double() * decay - Xo[i].double()
            bound = 2e-2 * (upd_ref.norm() / Xo[i].double().norm()).item() + 4e-3
            e = rel_fro(p.detach(), Xo[i])
            worst = max(worst, e / bound)
            assert e <= bound, (step, i, e, bound)
        print(f"config 2 step {step}: worst error / bound = {worst:.3f}")
        for i, p in enumerate(params):   # keep the trajectories together through the bf16 noise
            p.data.copy_(Xo[i])


def test_config3_rank1_bf16_momentum_10_steps(dev):
    """Rank fraction 1.0 (r = 768) with bf16 weights and momentum, fp32 Q, on 768^2, 3072x768 and 768x3072: every
    product rounds to bf16, so the bar is bf16-level on M and X; Q stays column-normalised."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            assert st["momentum"].dtype == torch.bfloat16 and st["Q"].dtype == torch.float32
            assert st["Q"].shape == (768, 768)
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            print(f"config 3 r=768 bf16 step {step} matrix {i}: M {eM:.2e} X {eX:.2e}")
            assert eM <= 1e-2 and eX <= 1e-2, (step, i, eM, eX)
            assert (st["Q"].double().norm(dim=0) - 1).abs().max().item() < 1e-2
        info = torch.cat([v for v in opt.cholesky_info().values()])
        assert int(info.abs().sum().item()) == 0

    _run_dion(dev, [(768, 768), (3072, 768), (768, 3072)], 1.0, 10, torch.bfloat16, torch.bfloat16, torch.float32,
              check=check)


def test_config3_rank1_fp32_state_incl_tall(dev):
    """The same three shapes at r = 768 in all-fp32 state: M and X within 1e-4; Q is conditioning-limited for the
    square matrix (the reference's own fp32-vs-fp64 spread there is 7e-4)."""
    def check(step, params, opt, Xo, Mo, Qo):
        for i, p in enumerate(params):
            st = opt.state[p]
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            eQ = rel_fro(_sign_align(st["Q"].cpu(), Qo[i]), Qo[i])
            print(f"config 3 r=768 fp32 step {step} matrix {i}: M {eM:.2e} X {eX:.2e} Q {eQ:.2e}")
            assert eM <= 1e-4 and eX <= 1e-4, (step, i, eM, eX)
            assert eQ <= (5e-3 if p.shape[0] == p.shape[1] else 3e-4)

    _run_dion(dev, [(768, 768), (3072, 768), (768, 3072)], 1.0, 4, torch.float32, torch.float32, torch.float32,
              check=check)


def test_config4_llama8b_layer_muon_step(dev):
    """One whole Llama-3-8B layer (7 bf16 matrices, four shape buckets in grouped launches) through `Muon.step()`:
    momentum bit exact; the Newton-Schulz result of every matrix against the oracle's on the same bf16 input
    (<= 2e-2 relative Frobenius); weights within that bar."""
    from dion_amd import Muon, zeropower_via_newtonschulz5
    from oracle import muon_step as O
    from oracle.newton_schulz import ns5

    shapes = LLAMA8B_LAYER
    gen = torch.Generator(device=dev).manual_seed(4)
    X0 = [(torch.randn(s, generator=gen, device=dev) * 0.02).bfloat16().cpu() for s in shapes]
    G = [(torch.randn(s, generator=gen, device=dev) * 1e-3).bfloat16().cpu() for s in shapes]
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    for p, g in zip(params, G):
        p.grad = g.to(dev)
    lr, mu, wd = 0.02, 0.95, 0.01
    opt = Muon(params, lr=lr, mu=mu, weight_decay=wd, nesterov=True, adjust_lr="spectral_norm")
    opt.step()
    torch.cuda.synchronize()
    lr_t, mu_t, wd_t = torch.tensor(lr), torch.tensor(mu), torch.tensor(wd)
    decay = (1 - lr_t * wd_t).item()
    seen = set()
    for i, (x0, g, p) in enumerate(zip(X0, G, params)):
        m = torch.zeros_like(x0)
        U = O.muon_pre([g], [m], mu_t, True)[0]
        assert torch.equal(opt.state[p]["momentum"].cpu(), m), f"momentum differs, matrix {i}"
        ns_ref = ns5(U, epsilon=torch.tensor(1e-8))
        if x0.shape not in seen:   # the orthogonalisation itself, once per shape
            seen.add(x0.shape)
            e_ns = rel_fro(zeropower_via_newtonschulz5(U.to(dev), epsilon=1e-8), ns_ref)
            print(f"config 4 NS {tuple(x0.shape)}: rel. Frobenius error {e_ns:.2e}")
            assert e_ns <= 2e-2
        xo = x0.clone()
        O.muon_post([xo], [ns_ref], lr_t, O.adjust_lr(lr_t, x0.shape, "spectral_norm"), wd_t)
        upd_ref = x0.double() * decay - xo.double()
        bound = 2e-2 * (upd_ref.norm() / xo.double().norm()).item() + 4e-3
        e = rel_fro(p.detach(), xo)
        print(f"config 4 weights {tuple(x0.shape)}: {e:.2e} (bound {bound:.2e})")
        assert e <= bound


def test_config5_llama70b_mlp_dion_5_steps(dev):
    """28672x8192 (a two-matrix bucket) and 8192x28672 under Dion with r = 512, bf16 weights / momentum, fp32 Q,
    5 consecutive steps so that the error feedback accumulates, against the oracle after every step."""
    from dion_amd import Dion, DionMixedPrecisionConfig
    from oracle import dion_step as O

    shapes = [(28672, 8192), (28672, 8192), (8192, 28672)]
    gen = torch.Generator(device=dev).manual_seed(5)
    X0 = [(torch.randn(s, generator=gen, device=dev) * 0.02).bfloat16() for s in shapes]
    gq = torch.Generator().manual_seed(2)
    Q0 = []
    for _ in shapes:
        q = torch.randn((8192, 512), generator=gq)
        Q0.append(q / q.norm(dim=0, keepdim=True))
    params = [torch.nn.Parameter(x.clone()) for x in X0]
    opt = Dion(params, rank_fraction=1.0 / 16, lr=0.01, mu=0.95, weight_decay=0.01,
               mixed_precision_config=DionMixedPrecisionConfig(momentum_dtype=torch.bfloat16, Q_dtype=torch.float32))
    Xo = [x.cpu() for x in X0]
    Mo = [torch.zeros_like(x) for x in Xo]
    Qo = [q.clone() for q in Q0]
    sk = torch.Generator().manual_seed(0)
    for step in range(5):
        Gd = [(torch.randn(s, generator=gen, device=dev) * 1e-3).bfloat16() for s in shapes]
        for p, g in zip(params, Gd):
            p.grad = g
        if step == 0:
            for p, q in zip(params, Q0):
                st = opt._get_or_initialize_state(p, opt.param_groups[0])
                assert st["Q"].shape == (8192, 512)
                st["Q"].copy_(q.to(dev))
        opt.step()
        O.dion_step(Xo, [g.cpu() for g in Gd], Mo, Qo, lr=0.01, mu=0.95, weight_decay=0.01, generator=sk)
        torch.cuda.synchronize()
        for i, p in enumerate(params):
            st = opt.state[p]
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            qn = (st["Q"].double().norm(dim=0) - 1).abs().max().item()
            print(f"config 5 step {step} matrix {i} {tuple(p.shape)}: M {eM:.2e} X {eX:.2e} | |Q col| - 1 {qn:.1e}",
                  flush=True)
            assert eM <= 1e-2 and eX <= 1e-2, (step, i, eM, eX)
            assert qn < 1e-2
        info = torch.cat([v for v in opt.cholesky_info().values()])
        assert int(info.abs().sum().item()) == 0


@pytest.mark.parametrize("bad", [float("nan"), float("inf")])
def test_dion_non_finite_gradient_follows_the_reference_guard(dev, bad):
    """One NaN / Inf in a gradient (reference dion/dion.py:1416-1444 `fix_all_zero_or_nan`): the factors are
    `nan_to_num`'d to zero, so M keeps B (with the bad entry), Q becomes 0 / (0 + eps) = 0 and X only decays --
    and the other matrix of the bucket is untouched by its neighbour's bad value."""
    from dion_amd import Dion
    from oracle import dion_step as O

    torch.manual_seed(0)
    shapes = [(256, 128), (256, 128)]
    X0 = [torch.randn(s) * 0.02 for s in shapes]
    G = [torch.randn(s) * 1e-3 for s in shapes]
    G[0][17, 5] = bad
    Q0 = [torch.randn(128, 32) for _ in shapes]
    Xo, Mo, Qo = [x.clone() for x in X0], [torch.zeros_like(x) for x in X0], [q.clone() for q in Q0]
    O.dion_step(Xo, G, Mo, Qo, lr=0.01, mu=0.95, weight_decay=0.01)
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    for p, g in zip(params, G):
        p.grad = g.to(dev)
    opt = Dion(params, rank_fraction=0.25, lr=0.01, mu=0.95, weight_decay=0.01)
    for p, q in zip(params, Q0):
        opt._get_or_initialize_state(p, opt.param_groups[0])["Q"].copy_(q.to(dev))
    opt.step()
    torch.cuda.synchronize()
    # the clean matrix: ordinary parity
    st1 = opt.state[params[1]]
    assert rel_fro(st1["momentum"], Mo[1]) <= 1e-4 and rel_fro(params[1].detach(), Xo[1]) <= 1e-4
    # the matrix with the bad gradient entry: same non-finite pattern in M, same finite values elsewhere
    m_got, m_ref = opt.state[params[0]]["momentum"].cpu(), Mo[0]
    assert torch.equal(torch.isfinite(m_got), torch.isfinite(m_ref))
    fin = torch.isfinite(m_ref)
    assert torch.allclose(m_got[fin], m_ref[fin], rtol=1e-5, atol=1e-9)
    assert torch.isfinite(params[0].detach()).all() and torch.isfinite(Xo[0]).all()
    assert torch.allclose(params[0].detach().cpu(), Xo[0], rtol=1e-6, atol=1e-9)
    q_got = opt.state[params[0]]["Q"].cpu()
    assert torch.isfinite(q_got).all() and torch.isfinite(Qo[0]).all()
    assert torch.allclose(q_got, Qo[0], rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("rank_fraction", [0.25, 1.0])
def test_config3_full_72_matrix_dion_step(dev, rank_fraction):
    """All 72 GPT-small matrices (buckets of 48 / 12 / 12 on three streams, the calls of a wave enqueued by worker
    threads: the default path of `Dion.step`) with bf16 weights and momentum and fp32 Q, 10 consecutive steps against
    `oracle.dion_step` (reference dion/dion.py:742-875).

    Two optimizers run side by side.  `free` follows its own trajectory (bar 1e-2 on M and X, the bf16 level).  `sync`
    is put back on the oracle's state after every step, so that a step's *update* can be compared sharply: one step
    moves X by less than 1 % of its norm, which the bar on X itself cannot see.  Measured on the updates:
      error feedback  (M_new - B) = -(1 - mu) P R^T, B = M + G (bit exact)   measured <= 1.0e-2, bar 2e-2
      weight update   (X_new - X)         measured <= 2.6e-2 (r = 192) / 7.8e-2 (r = 768), bar 5e-2 / 1.2e-1
    (both are differences of bf16 values: the weight update is 1-2 ulps of a weight, and a different summation order
    inside the rank-r products flips the rounding of some of them; a wrong scale, sign or operand is an error of 1)."""
    from dion_amd import Dion, DionMixedPrecisionConfig
    from oracle import dion_step as O

    shapes = GPT_SMALL_LAYER * 12
    bf = torch.bfloat16
    g0 = torch.Generator().manual_seed(11)
    X0 = [(torch.randn(s, generator=g0) * 0.02).to(bf) for s in shapes]
    gq = torch.Generator().manual_seed(2)
    Q0 = []
    for (m, n) in shapes:
        q = torch.randn((min(m, n), O.rank_of(m, n, rank_fraction)), generator=gq)
        Q0.append(q / q.norm(dim=0, keepdim=True))
    mp = DionMixedPrecisionConfig(momentum_dtype=bf, Q_dtype=torch.float32)
    opts, plists = [], []
    for _ in range(2):
        params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
        opt = Dion(params, rank_fraction=rank_fraction, lr=0.01, mu=0.95, weight_decay=0.01, mixed_precision_config=mp)
        for p, q in zip(params, Q0):
            opt._get_or_initialize_state(p, opt.param_groups[0])["Q"].copy_(q.to(dev))
        opts.append(opt)
        plists.append(params)
    (sync, free), (ps, pf) = opts, plists
    Xo, Mo, Qo = [x.clone() for x in X0], [torch.zeros_like(x) for x in X0], [q.clone() for q in Q0]
    gg = torch.Generator().manual_seed(3)
    sk = torch.Generator().manual_seed(0)
    worst = dict(ef=0.0, dx=0.0, M=0.0, X=0.0)
    for step in range(10):
        G = [(torch.randn(s, generator=gg) * 1e-3).to(bf) for s in shapes]
        for params in plists:
            for p, g in zip(params, G):
                p.grad = g.to(dev)
        Xprev = [x.clone() for x in Xo]
        B = [m + g for m, g in zip(Mo, G)]                      # bf16 add, as torch._foreach_add_ (dion.py:794)
        sync.step()
        free.step()
        O.dion_step(Xo, G, Mo, Qo, lr=0.01, mu=0.95, weight_decay=0.01, generator=sk)
        torch.cuda.synchronize()
        for opt in opts:
            info = torch.cat([v for v in opt.cholesky_info().values()])
            assert info.numel() == 72 and int(info.abs().sum().item()) == 0, f"step {step}: info {info.tolist()}"
        for i in range(72):
            st = sync.state[ps[i]]
            ef_ref = Mo[i].double() - B[i].double()
            ef_got = st["momentum"].cpu().double() - B[i].double()
            dx_ref = Xo[i].double() - Xprev[i].double()
            dx_got = ps[i].detach().cpu().double() - Xprev[i].double()
            e_ef = ((ef_got - ef_ref).norm() / ef_ref.norm()).item()
            e_dx = ((dx_got - dx_ref).norm() / dx_ref.norm()).item()
            worst["ef"], worst["dx"] = max(worst["ef"], e_ef), max(worst["dx"], e_dx)
            assert e_ef <= 2e-2 and e_dx <= (5e-2 if rank_fraction < 1 else 1.2e-1), (step, i, shapes[i], e_ef, e_dx)
            assert (st["Q"].double().norm(dim=0) - 1).abs().max().item() < 1e-2
            eM, eX = rel_fro(free.state[pf[i]]["momentum"], Mo[i]), rel_fro(pf[i].detach(), Xo[i])
            worst["M"], worst["X"] = max(worst["M"], eM), max(worst["X"], eX)
            assert eM <= 1e-2 and eX <= 1e-2, (step, i, shapes[i], eM, eX)
            # back onto the oracle's state
            ps[i].data.copy_(Xo[i])
            st["momentum"].copy_(Mo[i])
            st["Q"].copy_(Qo[i])
        print(f"config 3, 72 matrices, rank fraction {rank_fraction}, step {step}: worst so far {worst}", flush=True)
