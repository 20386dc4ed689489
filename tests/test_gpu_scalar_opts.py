"""GPU parity of the fused Lion / AdamW passes (`dion_amd_lion_step`, `dion_amd_adamw_step`) against the CPU
oracle (reference dion/scalar_opts.py:89-187)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

BF, F32 = torch.bfloat16, torch.float32
SIZES = [1, 7, 8, 1000, 4099, 50304 * 8]


def _close(got, want, what, operand=None, ulps=1):
    """Element-wise ops in the reference's rounding sequence: equal but for last-bit effects -- the CPU's scalar tail
    path does not fuse the multiply-add of lerp, and its vectorised fp32 sqrt is not correctly rounded (the kernel's
    is: it equals sqrt evaluated in fp64, and PyTorch's own GPU ops, bit for bit).  Never more than one unit in the
    last place of the result or of the `operand` it was formed from by a subtraction (`ulps` of them where a
    1-ulp difference of the square root passes through a division and two more roundings)."""
    got, want = got.detach().cpu(), want.detach()
    assert got.dtype == want.dtype and got.shape == want.shape
    g, w = got.double(), want.double()
    ulp = 2.0 ** -7 if got.dtype == BF else 2.0 ** -22
    mag = w.abs() if operand is None else torch.maximum(w.abs(), operand.double().abs())
    assert torch.all((g - w).abs() <= ulps * ulp * mag.clamp_min(1e-30) + 1e-38), f"{what}: more than {ulps} ulp"
    if got.numel() >= 1000:  # short tensors run wholly on the CPU's unfused scalar path
        assert (g != w).double().mean().item() <= 2e-2, f"{what}: too many last-bit differences"


def _problem(dtypes, seed, sizes=SIZES, unaligned=False):
    xd, gd, md, vd = dtypes
    gen = torch.Generator().manual_seed(seed)
    mk = lambda n, s, d: (torch.randn(n + 1, generator=gen) * s).to(d)[1 if unaligned else 0:][:n]  # noqa: E731
    X = [mk(n, 1.0, xd) for n in sizes]
    G = [mk(n, 0.1, gd) for n in sizes]
    M = [mk(n, 0.1, md) for n in sizes]
    V = [(mk(n, 0.1, F32) ** 2).to(vd) for n in sizes]
    return X, G, M, V


def _hyper():
    t = lambda z: torch.tensor(z)  # noqa: E731
    return dict(lr=t(0.01), beta1=t(0.9), beta2=t(0.95), weight_decay=t(0.1))


@pytest.mark.parametrize("dtypes", [(BF, BF, BF, BF), (F32, F32, F32, F32), (BF, BF, F32, F32), (F32, BF, F32, BF)])
@pytest.mark.parametrize("unaligned", [False, True])
def test_lion_matches_oracle(dev, dtypes, unaligned):
    from dion_amd.elementwise_opts import lion_update_foreach
    from oracle import scalar_opts as O

    sizes = SIZES[:-1] if unaligned else SIZES
    X, G, M, _ = _problem(dtypes, 5, sizes, unaligned)
    Xd, Gd, Md = ([t.to(dev) for t in L] for L in (X, G, M))
    if unaligned:  # .to(dev) makes fresh, aligned storage: slice again on the device
        Xd, Gd, Md = ([torch.cat([t[:1], t])[1:] for t in L] for L in (Xd, Gd, Md))
    Xo, Mo = [t.clone() for t in X], [t.clone() for t in M]
    for _ in range(2):
        O.lion_update_foreach(Xo, G, Mo, **_hyper())
        lion_update_foreach(Xd, Gd, Md, **_hyper())
    for i, n in enumerate(sizes):
        _close(Md[i], Mo[i], f"momentum n={n}")
        _close(Xd[i], Xo[i], f"weights n={n}", operand=X[i])


@pytest.mark.parametrize("dtypes", [(BF, BF, BF, BF), (F32, F32, F32, F32), (BF, BF, F32, F32), (F32, BF, F32, BF)])
@pytest.mark.parametrize("unaligned", [False, True])
def test_adamw_matches_oracle(dev, dtypes, unaligned):
    from dion_amd.elementwise_opts import adamw_update_foreach
    from oracle import scalar_opts as O

    sizes = SIZES[:-1] if unaligned else SIZES
    X, G, M, V = _problem(dtypes, 6, sizes, unaligned)
    Xd, Gd, Md, Vd = ([t.to(dev) for t in L] for L in (X, G, M, V))
    if unaligned:
        Xd, Gd, Md, Vd = ([torch.cat([t[:1], t])[1:] for t in L] for L in (Xd, Gd, Md, Vd))
    Xo, Mo, Vo = [t.clone() for t in X], [t.clone() for t in M], [t.clone() for t in V]
    for step in (1, 2, 3):
        prev = [t.clone() for t in Xo]
        O.adamw_update_foreach(Xo, G, Mo, Vo, step=torch.tensor(step), epsilon=torch.tensor(1e-8), **_hyper())
        adamw_update_foreach(Xd, Gd, Md, Vd, step=torch.tensor(step), epsilon=torch.tensor(1e-8), **_hyper())
        # keep the trajectories together: a last-bit difference in V near zero is amplified by 1/sqrt(V)
        for k, (a, b) in enumerate(zip((Xd, Md, Vd), (Xo, Mo, Vo))):
            for i, n in enumerate(sizes):
                _close(a[i], b[i], f"step {step} n={n} {'XMV'[k]}", operand=(prev[i].double().abs() + (prev[i].double() - Xo[i].double()).abs()) if k == 0 else None,
                       ulps=3 if k == 0 else 1)
                a[i].copy_(b[i])


def test_many_tensors_and_argument_errors(dev):
    """More tensors than one launch's table holds; empty tensors; CPU tensors and mismatched shapes are refused."""
    from dion_amd import _lib
    from dion_amd.elementwise_opts import lion_update_foreach
    from oracle import scalar_opts as O

    sizes = [17 + 3 * i for i in range(110)] + [0]
    X, G, M, _ = _problem((F32, F32, F32, F32), 7, sizes)
    Xd, Gd, Md = ([t.to(dev) for t in L] for L in (X, G, M))
    O.lion_update_foreach(X, G, M, **_hyper())
    lion_update_foreach(Xd, Gd, Md, **_hyper())
    for i, n in enumerate(sizes):
        _close(Md[i], M[i], f"momentum n={n}")
        _close(Xd[i], X[i], f"weights n={n}", operand=X[i] + 1.0)
    with pytest.raises(_lib.DionAmdError):
        lion_update_foreach([X[0]], [G[0]], [M[0]], **_hyper())            # CPU tensors: no fallback
    with pytest.raises(_lib.DionAmdError):
        lion_update_foreach([Xd[0]], [Gd[1]], [Md[0]], **_hyper())         # shapes differ
    with pytest.raises(_lib.DionAmdError):
        lion_update_foreach([Xd[3].double()], [Gd[3].double()], [Md[3].double()], **_hyper())  # unsupported dtype
