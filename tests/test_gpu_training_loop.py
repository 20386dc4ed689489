"""The optimizers inside an ordinary training loop (reference train.py:311-337, 363-377, 416-425, 919-920): autograd
gradients, the three-group layout of the reference's `init_optimizer` (matrices -> Muon / Dion, embedding and lm_head ->
Lion with lm_head at lr / sqrt(d), gains and biases -> AdamW) and a learning-rate scheduler that rewrites `group["lr"]`
before every step.  The same loop runs on the CPU with the oracle's step functions; the loss curves must agree."""
import math

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

V, D, H, BATCH, STEPS = 96, 64, 256, 512, 12


def _init(seed):
    g = torch.Generator().manual_seed(seed)
    return dict(
        emb=torch.randn(V, D, generator=g) * 0.5,
        fc=torch.randn(H, D, generator=g) * (1 / math.sqrt(D)),
        proj=torch.randn(D, H, generator=g) * (1 / math.sqrt(H)),
        head=torch.randn(V, D, generator=g) * 0.1,
        gain=torch.ones(D),
        bias=torch.zeros(D),
    )


def _loss(p, tokens, targets):
    h = p["emb"][tokens] * p["gain"]
    h = h + F.gelu(h @ p["fc"].T) @ p["proj"].T + p["bias"]
    return F.cross_entropy(h @ p["head"].T, targets)


def _data(seed):
    g = torch.Generator().manual_seed(seed)
    tokens = torch.randint(0, V, (BATCH,), generator=g)
    return tokens, (tokens * 7 + 3) % V   # a fixed map of the token: learnable by this model


def _schedule(step):
    return 1.0 - 0.5 * step / STEPS


def _oracle_loop(kind, q0):
    from oracle import dion_step as OD
    from oracle import muon_step as OM
    from oracle import scalar_opts as OS

    p = {k: v.clone().requires_grad_(True) for k, v in _init(0).items()}
    tokens, targets = _data(1)
    lr0, mu, wd = 0.02, 0.95, 0.01
    mats = [p["fc"], p["proj"]]
    Mm = [torch.zeros_like(x) for x in mats]
    Q = [q.clone() for q in q0] if kind == "dion" else None
    lion = [(p["emb"], lr0), (p["head"], lr0 / math.sqrt(D))]
    Ml = [torch.zeros_like(x) for x, _ in lion]
    adam = [p["gain"], p["bias"]]
    Ma, Va = [torch.zeros_like(x) for x in adam], [torch.zeros_like(x) for x in adam]
    sketch = torch.Generator().manual_seed(0)
    losses = []
    for step in range(STEPS):
        loss = _loss(p, tokens, targets)
        grads = torch.autograd.grad(loss, list(p.values()))
        G = dict(zip(p.keys(), grads))
        losses.append(loss.item())
        f = _schedule(step)
        with torch.no_grad():
            gm = [G["fc"], G["proj"]]
            if kind == "muon":
                OM.muon_step([x.data for x in mats], gm, Mm, lr=lr0 * f, mu=mu, weight_decay=wd, epsilon=1e-8,
                             nesterov=True)
            else:
                OD.dion_step([x.data for x in mats], gm, Mm, Q, lr=lr0 * f, mu=mu, weight_decay=wd, generator=sketch)
            for (x, lr), m, name in zip(lion, Ml, ("emb", "head")):
                OS.lion_update_foreach([x.data], [G[name]], [m], lr=torch.tensor(lr * f), beta1=torch.tensor(0.9),
                                       beta2=torch.tensor(0.95), weight_decay=torch.tensor(wd))
            OS.adamw_update_foreach([x.data for x in adam], [G["gain"], G["bias"]], Ma, Va, lr=torch.tensor(lr0 * f),
                                    beta1=torch.tensor(0.9), beta2=torch.tensor(0.95), weight_decay=torch.tensor(0.0),
                                    step=torch.tensor(step + 1), epsilon=torch.tensor(1e-8))
    return losses


@pytest.mark.parametrize("kind", ["muon", "dion"])
def test_training_loop_follows_the_oracle(dev, kind):
    from dion_amd import Dion, Muon
    from oracle import dion_step as OD

    p = {k: torch.nn.Parameter(v.clone().to(dev)) for k, v in _init(0).items()}
    tokens, targets = (t.to(dev) for t in _data(1))
    lr0, mu, wd = 0.02, 0.95, 0.01
    groups = [
        dict(params=[p["fc"], p["proj"]]),
        dict(params=[p["emb"]], algorithm="lion"),
        dict(params=[p["head"]], algorithm="lion", lr=lr0 / math.sqrt(D)),
        dict(params=[p["gain"], p["bias"]], algorithm="adamw", weight_decay=0.0),
    ]
    q0 = None
    if kind == "muon":
        opt = Muon(groups, lr=lr0, mu=mu, weight_decay=wd, nesterov=True)
    else:
        opt = Dion(groups, lr=lr0, mu=mu, weight_decay=wd, rank_fraction=0.5)
        gq = torch.Generator().manual_seed(2)
        q0 = []
        for x in (p["fc"], p["proj"]):
            m, n = x.shape
            q0.append(torch.randn((m if m < n else n, OD.rank_of(m, n, 0.5)), generator=gq))
            opt._get_or_initialize_state(x, opt.param_groups[0])["Q"].copy_(q0[-1].to(dev))
    sched = torch.optim.lr_scheduler.LambdaLR(opt, _schedule)
    losses = []
    for step in range(STEPS):
        opt.zero_grad(set_to_none=True)
        loss = _loss(p, tokens, targets)
        loss.backward()
        losses.append(loss.item())
        opt.step()
        sched.step()
    ref = _oracle_loop(kind, q0)
    print(kind, "gpu", [f"{v:.4f}" for v in losses])
    print(kind, "cpu", [f"{v:.4f}" for v in ref])
    assert all(g["step"] == STEPS for g in opt.param_groups)
    assert losses[-1] < 0.8 * losses[0], "the loop does not train"
    # all-fp32 Dion tracks the oracle to rounding; Muon's bf16 Newton-Schulz carries 1e-2 of noise per update
    tol = 2e-3 if kind == "dion" else 2e-2
    for step, (a, b) in enumerate(zip(losses, ref)):
        assert abs(a - b) <= tol * abs(b), (step, a, b)
