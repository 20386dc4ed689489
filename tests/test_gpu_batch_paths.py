"""The roads through the library that depend on the batch: bit-level comparisons on the GPU alone.

  * error feedback + weight update as one pass vs. as two products (reference dion/dion.py:851-853, 865-872);
  * `Dion.step` with its buckets enqueued by worker threads on three streams vs. one after the other;
  * a matrix inside a bucket of the benchmark's size vs. the same matrix stepped alone (reference dion/muon.py:356-486
    and dion/dion.py:742-875 treat every matrix of a batch independently);
  * the Muon weight update inside the epilogue of the last Newton-Schulz product vs. as the stand-alone pass behind a
    stand-alone orthogonalisation (reference dion/muon.py:568-573).
"""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

BF = torch.bfloat16


def _dion_problem(dev, shapes, seed, scale_x=0.02):
    gen = torch.Generator(device=dev).manual_seed(seed)
    X = [(torch.randn(s, generator=gen, device=dev) * scale_x).to(BF) for s in shapes]
    return X, gen


def _make_dion(dev, X, rank_fraction, Q=None):
    from dion_amd import Dion, DionMixedPrecisionConfig

    params = [torch.nn.Parameter(x.clone()) for x in X]
    opt = Dion(params, rank_fraction=rank_fraction, lr=0.01, mu=0.95, weight_decay=0.01,
               mixed_precision_config=DionMixedPrecisionConfig(momentum_dtype=BF, Q_dtype=torch.float32))
    states = [opt._get_or_initialize_state(p, opt.param_groups[0]) for p in params]
    if Q is not None:
        for st, q in zip(states, Q):
            st["Q"].copy_(q)
    return opt, params, states


def _assert_same(tag, pa, sa, pb, sb):
    for i, (a, b) in enumerate(zip(pa, pb)):
        assert torch.equal(a.detach(), b.detach()), f"{tag}: X differs, matrix {i}"
        assert torch.equal(sa[i]["momentum"], sb[i]["momentum"]), f"{tag}: M differs, matrix {i}"
        assert torch.equal(sa[i]["Q"], sb[i]["Q"]), f"{tag}: Q differs, matrix {i}"


@pytest.mark.parametrize("shapes,rank_fraction", [
    ([(768, 768)] * 3 + [(3072, 768)] * 2 + [(768, 3072)] * 2, 0.25),
    ([(768, 768)] * 3 + [(3072, 768)] * 2 + [(768, 3072)] * 2, 1.0),
    ([(28672, 8192)] * 2, 1.0 / 16),
    ([(8192, 28672)] * 2, 1.0 / 16),
])
def test_fused_update_pass_equals_the_two_products_bit_for_bit(dev, shapes, rank_fraction):
    """`dion_ef_update_kernel` (one pass over M and X) against the two AXPBY products it replaces, switched per
    process with `dion_amd_set_option("fused_update", ...)`: M, X and Q after two steps, `torch.equal`."""
    from dion_amd import _lib

    X, gen = _dion_problem(dev, shapes, 21)
    G = [[(torch.randn(s, generator=gen, device=dev) * 1e-3).to(BF) for s in shapes] for _ in range(2)]
    runs = []
    try:
        for fused in (1, 0):
            _lib.set_option("fused_update", fused)
            torch.manual_seed(5)
            opt, params, states = _make_dion(dev, X, rank_fraction)
            if runs:
                for st, ref in zip(states, runs[0][3]):
                    st["Q"].copy_(ref)
            q0 = [st["Q"].clone() for st in states]
            for step in range(2):
                for p, g in zip(params, G[step]):
                    p.grad = g
                opt.step()
            torch.cuda.synchronize()
            assert all(int(v.abs().sum().item()) == 0 for v in opt.cholesky_info().values())
            runs.append((opt, params, states, q0))
    finally:
        _lib.set_option("fused_update", -1)
    _assert_same("one pass vs two products", runs[0][1], runs[0][2], runs[1][1], runs[1][2])
    # and the step did something: the weights moved
    assert not torch.equal(runs[0][1][0].detach(), X[0])


def test_dion_step_serial_and_threaded_enqueue_give_the_same_bits(dev, monkeypatch):
    """Three buckets: once with the default path (one worker thread and stream per bucket of a wave), once with
    DION_AMD_DION_SERIAL=1 (the caller's thread, one call after the other; also what runs under stream capture)."""
    shapes = [(768, 768)] * 8 + [(3072, 768)] * 3 + [(768, 3072)] * 3 + [(256, 512)] * 2
    X, gen = _dion_problem(dev, shapes, 33)
    G = [[(torch.randn(s, generator=gen, device=dev) * 1e-3).to(BF) for s in shapes] for _ in range(3)]
    runs = []
    for serial in (False, True):
        if serial:
            monkeypatch.setenv("DION_AMD_DION_SERIAL", "1")
        else:
            monkeypatch.delenv("DION_AMD_DION_SERIAL", raising=False)
        opt, params, states = _make_dion(dev, X, 0.25)
        if runs:
            for st, ref in zip(states, runs[0][3]):
                st["Q"].copy_(ref)
        q0 = [st["Q"].clone() for st in states]
        for step in range(3):
            for p, g in zip(params, G[step]):
                p.grad = g
            opt.step()
        torch.cuda.synchronize()
        runs.append((opt, params, states, q0))
    _assert_same("threaded vs serial", runs[0][1], runs[0][2], runs[1][1], runs[1][2])


@pytest.mark.parametrize("shape", [(4096, 4096), (4096, 14336), (14336, 4096)])
def test_muon_matrix_in_a_64_matrix_bucket_equals_the_matrix_alone(dev, shape):
    """Llama-3-8B bucket sizes of the benchmark (64 matrices of 4096^2 resp. 4096 x 14336 per shape): matrix 37 of
    the bucket and the same matrix as a bucket of its own, momentum and weights bit for bit."""
    from dion_amd import Muon

    pick, nb = 37, 64
    gen = torch.Generator(device=dev).manual_seed(4)
    X = [(torch.randn(shape, generator=gen, device=dev) * 0.02).to(BF) for _ in range(nb)]
    G = [(torch.randn(shape, generator=gen, device=dev) * 1e-3).to(BF) for _ in range(nb)]
    kw = dict(lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True, adjust_lr="spectral_norm")
    whole = [torch.nn.Parameter(x.clone()) for x in X]
    for p, g in zip(whole, G):
        p.grad = g
    alone = torch.nn.Parameter(X[pick].clone())
    alone.grad = G[pick].clone()
    opt_w, opt_a = Muon(whole, **kw), Muon([alone], **kw)
    opt_w.step()
    opt_a.step()
    torch.cuda.synchronize()
    assert torch.equal(opt_w.state[whole[pick]]["momentum"], opt_a.state[alone]["momentum"])
    assert torch.equal(whole[pick].detach(), alone.detach())
    assert not torch.equal(alone.detach(), X[pick])


def test_dion_matrix_in_a_16_matrix_70b_bucket(dev):
    """The 16-matrix 28672 x 8192 bucket of the Llama-3-70B workload at r = 512.  The products of a Dion step choose
    how many slices to cut their sums into from the size of the batch, so a matrix stepped alone may differ from
    itself inside the bucket in the last bit of a sum; what must hold exactly is independence from the neighbours:
    the bucket in another order gives the same bits per matrix.  Against the matrix alone: bf16 level."""
    from conftest import rel_fro

    shape, nb, pick = (28672, 8192), 16, 11
    X, gen = _dion_problem(dev, [shape] * nb, 5)
    G = [(torch.randn(shape, generator=gen, device=dev) * 1e-3).to(BF) for _ in range(nb)]
    torch.manual_seed(2)
    opt, params, states = _make_dion(dev, X, 1.0 / 16)
    Q0 = [st["Q"].clone() for st in states]
    perm = [(i * 5 + 3) % nb for i in range(nb)]          # a permutation of 0..15 (5 and 16 are coprime)
    opt_p, params_p, states_p = _make_dion(dev, [X[j] for j in perm], 1.0 / 16, [Q0[j] for j in perm])
    opt_1, params_1, states_1 = _make_dion(dev, [X[pick]], 1.0 / 16, [Q0[pick]])
    for step in range(2):
        for p, g in zip(params, G):
            p.grad = g
        for p, j in zip(params_p, perm):
            p.grad = G[j]
        params_1[0].grad = G[pick]
        opt.step()
        opt_p.step()
        opt_1.step()
    torch.cuda.synchronize()
    for k, j in enumerate(perm):
        assert torch.equal(params_p[k].detach(), params[j].detach()), f"X of matrix {j} depends on its position"
        assert torch.equal(states_p[k]["momentum"], states[j]["momentum"]), f"M of matrix {j} depends on its position"
        assert torch.equal(states_p[k]["Q"], states[j]["Q"]), f"Q of matrix {j} depends on its position"
    eM = rel_fro(states_1[0]["momentum"], states[pick]["momentum"])
    eX = rel_fro(params_1[0].detach(), params[pick].detach())
    eQ = rel_fro(states_1[0]["Q"], states[pick]["Q"])
    print(f"70B bucket, matrix {pick} alone vs in the bucket: M {eM:.2e} X {eX:.2e} Q {eQ:.2e}")
    assert eM <= 2e-3 and eX <= 2e-4 and eQ <= 2e-3


@pytest.mark.parametrize("shapes,rank_fraction", [
    ([(768, 768)] * 5 + [(3072, 768)] * 3 + [(768, 3072)] * 3, 0.25),     # one column tile of P (r = 192)
    ([(1024, 512)] * 3 + [(512, 1024)] * 2, 0.07),                        # a rank off the 64-grid (r = 36 -> 40 columns)
    ([(28672, 8192)] * 2, 1.0 / 16),                                      # two column tiles, walked by one workgroup
    ([(8192, 28672)] * 2, 1.0 / 16),                                      # the same, B = M^T
])
def test_momentum_plus_gradient_inside_the_first_product_equals_the_separate_pass(dev, shapes, rank_fraction):
    """`B = M + G` formed inside the launch of `P = B Q` (dion_bq.hip) against the separate pass over M followed by the
    plain product (reference dion/dion.py:794, 801), switched with `dion_amd_set_option("fused_bq", ...)`: M, X and Q
    after three steps (the momentum is not zero from the second step on), `torch.equal`.  Matrix 0 starts with an
    all-zero B, which must take the all-zero guard (P = 0, R = Q: reference dion/dion.py:1416-1444) on both roads: a
    wrong non-zero flag would leave it with Q = 0."""
    from dion_amd import _lib

    X, gen = _dion_problem(dev, shapes, 33)
    G = [[(torch.randn(s, generator=gen, device=dev) * 1e-3).to(BF) for s in shapes] for _ in range(3)]
    G[0][0].zero_()      # matrix 0 starts with B = 0
    runs = []
    try:
        for fused in (1, 0):
            _lib.set_option("fused_bq", fused)
            torch.manual_seed(5)
            opt, params, states = _make_dion(dev, X, rank_fraction)
            if runs:
                for st, ref in zip(states, runs[0][3]):
                    st["Q"].copy_(ref)
            q0 = [st["Q"].clone() for st in states]
            for step in range(3):
                for p, g in zip(params, G[step]):
                    p.grad = g
                opt.step()
            torch.cuda.synchronize()
            runs.append((opt, params, states, q0))
    finally:
        _lib.set_option("fused_bq", -1)
    _assert_same("sum inside the product vs separate pass", runs[0][1], runs[0][2], runs[1][1], runs[1][2])
    assert not torch.equal(runs[0][1][1].detach(), X[1])


@pytest.mark.parametrize("wdtype", [BF, torch.float32])
@pytest.mark.parametrize("shapes", [
    [(768, 768)] * 2 + [(3072, 768)] * 2 + [(768, 3072)] * 2,      # product launches: square, tall (transposed), wide
    [(768, 768)] * 16 + [(3072, 768)] * 8 + [(768, 3072)] * 8,     # enough matrices for the persistent launch
])
def test_muon_update_in_the_last_epilogue_equals_the_stand_alone_pass(dev, shapes, wdtype):
    """`Muon.step` (momentum pass, Newton-Schulz whose last X' = aX + BX applies the weight update in its epilogue)
    against the same optimizer with the library's own orthogonalisation passed as `newton_schulz_func`, which makes
    the step run its three stages as separate calls (dion_amd_muon_pre, dion_amd_newton_schulz per matrix,
    dion_amd_muon_post): weights and momentum after two steps, bit for bit."""
    from dion_amd import Muon
    from dion_amd.newton_schulz import zeropower_via_newtonschulz5

    gen = torch.Generator(device=dev).manual_seed(11)
    X = [(torch.randn(s, generator=gen, device=dev) * 0.02).to(wdtype) for s in shapes]
    G = [[(torch.randn(s, generator=gen, device=dev) * 1e-3).to(wdtype) for s in shapes] for _ in range(2)]
    kw = dict(lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True, adjust_lr="spectral_norm")
    runs = []
    for hook in (None, zeropower_via_newtonschulz5):
        params = [torch.nn.Parameter(x.clone()) for x in X]
        opt = Muon(params, newton_schulz_func=hook, **kw)
        for step in range(2):
            for p, g in zip(params, G[step]):
                p.grad = g
            opt.step()
        torch.cuda.synchronize()
        runs.append((opt, params))
    (oa, pa), (ob, pb) = runs
    for i, (a, b) in enumerate(zip(pa, pb)):
        assert torch.equal(oa.state[a]["momentum"], ob.state[b]["momentum"]), f"momentum differs, matrix {i}"
        assert torch.equal(a.detach(), b.detach()), f"weights differ, matrix {i} {tuple(a.shape)}"
    assert not torch.equal(pa[0].detach(), X[0])
