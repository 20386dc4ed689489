"""Seeded random shapes, most of them off every alignment grid, through the three entry points that take matrices:
Newton-Schulz, a Muon step and Dion steps, each against the CPU oracle at the bar of its dtype."""
import random

import pytest
import torch

from conftest import rel_fro

pytestmark = pytest.mark.gpu


def _shapes(seed, count, lo, hi):
    rng = random.Random(seed)
    return [(rng.randint(lo, hi), rng.randint(lo, hi)) for _ in range(count)]


NS_SHAPES = [(1, 7), (3, 5), (5, 3), (8, 8), (9, 17), (255, 257), (129, 64)] + _shapes(7, 9, 10, 330)


@pytest.mark.parametrize("m,n", NS_SHAPES)
def test_ns_random_shapes(dev, m, n):
    from dion_amd import zeropower_via_newtonschulz5
    from oracle import newton_schulz as O

    torch.manual_seed(m * 1000 + n)
    G = torch.randn(3, m, n)
    ref = O.ns5(G)
    got = zeropower_via_newtonschulz5(G.to(dev))
    assert got.shape == (3, m, n) and got.dtype == torch.bfloat16
    for b in range(3):
        assert rel_fro(got[b], ref[b]) <= 2e-2, (m, n, b)


def test_muon_random_shapes(dev):
    from dion_amd import Muon
    from oracle import muon_step as O

    shapes = _shapes(11, 10, 9, 200)
    shapes += shapes[:3]   # buckets of two matrices
    g = torch.Generator().manual_seed(3)
    X0 = [torch.randn(s, generator=g) * 0.02 for s in shapes]
    Xo = [x.clone() for x in X0]
    Mo = [torch.zeros_like(x) for x in X0]
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    lr, mu, wd = 0.02, 0.9, 0.05
    opt = Muon(params, lr=lr, mu=mu, weight_decay=wd, nesterov=False, adjust_lr="rms_norm")
    for step in range(2):
        G = [torch.randn(s, generator=g) * 1e-3 for s in shapes]
        for p, gr in zip(params, G):
            p.grad = gr.to(dev)
        prev = [x.clone() for x in Xo]
        O.muon_step(Xo, G, Mo, lr=lr, mu=mu, weight_decay=wd, epsilon=1e-8, nesterov=False, adjust="rms_norm")
        opt.step()
        decay = (1 - torch.tensor(lr) * torch.tensor(wd)).item()
        for i, p in enumerate(params):
            assert torch.equal(opt.state[p]["momentum"].cpu(), Mo[i]), (shapes[i], step)
            upd_ref = prev[i].double() * decay - Xo[i].double()
            upd_got = prev[i].double() * decay - p.detach().cpu().double()
            assert rel_fro(upd_got, upd_ref) <= 2e-2, (shapes[i], step)
            p.data.copy_(Xo[i])


@pytest.mark.parametrize("seed,rank_fraction", [(21, 0.37), (22, 0.6), (23, 1.0)])
def test_dion_random_shapes(dev, seed, rank_fraction):
    from dion_amd import Dion, DionMixedPrecisionConfig
    from oracle import dion_step as O

    shapes = _shapes(seed, 6, 9, 260)
    if rank_fraction == 1.0:
        # full rank of a square-ish Gaussian matrix is conditioning-limited in Q; keep the aspect ratio >= 1.5
        shapes = [(m, n) for (m, n) in shapes if max(m, n) >= 1.5 * min(m, n)] or [(40, 120), (150, 60)]
    g = torch.Generator().manual_seed(seed)
    X0 = [torch.randn(s, generator=g) * 0.02 for s in shapes]
    Q0 = []
    for (m, n) in shapes:
        q = torch.randn((m if m < n else n, O.rank_of(m, n, rank_fraction)), generator=g)
        Q0.append(q / q.norm(dim=0, keepdim=True))
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    cfg = DionMixedPrecisionConfig(momentum_dtype=torch.float32, Q_dtype=torch.float32)
    opt = Dion(params, rank_fraction=rank_fraction, lr=0.01, mu=0.95, weight_decay=0.01, mixed_precision_config=cfg)
    Xo, Mo, Qo = [x.clone() for x in X0], [torch.zeros_like(x) for x in X0], [q.clone() for q in Q0]
    sk = torch.Generator().manual_seed(0)
    for step in range(3):
        G = [torch.randn(s, generator=g) * 1e-3 for s in shapes]
        for p, gr in zip(params, G):
            p.grad = gr.to(dev)
        if step == 0:
            for p, q in zip(params, Q0):
                st = opt._get_or_initialize_state(p, opt.param_groups[0])
                assert st["Q"].shape == q.shape
                st["Q"].copy_(q.to(dev))
        O.dion_step(Xo, G, Mo, Qo, lr=0.01, mu=0.95, weight_decay=0.01, generator=sk)
        opt.step()
        for i, p in enumerate(params):
            st = opt.state[p]
            eM, eX = rel_fro(st["momentum"], Mo[i]), rel_fro(p.detach(), Xo[i])
            s = torch.sign((st["Q"].cpu().double() * Qo[i].double()).sum(dim=0))
            s[s == 0] = 1
            eQ = rel_fro(st["Q"].cpu().double() * s, Qo[i])
            assert eM <= 1e-4 and eX <= 1e-4 and eQ <= 3e-4, (shapes[i], step, eM, eX, eQ)
        info = torch.cat([v for v in opt.cholesky_info().values()])
        assert int(info.abs().sum().item()) == 0
