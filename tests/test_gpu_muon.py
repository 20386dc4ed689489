"""GPU parity of `dion_amd.Muon.step()` against the CPU oracle (reference dion/muon.py:356-486)."""
import pytest
import torch

from conftest import rel_fro

pytestmark = pytest.mark.gpu

SHAPES_GPT_SMALL_LAYER = [(768, 768)] * 4 + [(3072, 768), (768, 3072)]


def _make(shapes, dtype, seed, gscale=1e-3):
    g = torch.Generator().manual_seed(seed)
    X = [(torch.randn(s, generator=g) * 0.02).to(dtype) for s in shapes]
    return X, g


def _grads(shapes, gen, dtype, gscale=1e-3):
    return [(torch.randn(s, generator=gen) * gscale).to(dtype) for s in shapes]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("nesterov", [True, False])
def test_muon_step_matches_oracle(dev, dtype, nesterov):
    from dion_amd import Muon
    from oracle import muon_step as O

    shapes = SHAPES_GPT_SMALL_LAYER * 2
    X0, gen = _make(shapes, dtype, seed=1)
    Xo = [x.clone() for x in X0]
    Mo = [torch.zeros_like(x) for x in X0]
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    lr, mu, wd = 0.02, 0.95, 0.01
    opt = Muon(params, lr=lr, mu=mu, weight_decay=wd, nesterov=nesterov, adjust_lr="spectral_norm")
    for step in range(3):
        G = _grads(shapes, gen, dtype)
        for p, g in zip(params, G):
            p.grad = g.to(dev)
        prev = [x.clone() for x in Xo]
        O.muon_step(Xo, G, Mo, lr=lr, mu=mu, weight_decay=wd, epsilon=1e-8, nesterov=nesterov)
        opt.step()
        for i, p in enumerate(params):
            mom = opt.state[p]["momentum"]
            assert mom.dtype == dtype and mom.shape == p.shape
            # the momentum pass is element-wise with the reference's rounding points: bit exact
            assert torch.equal(mom.cpu(), Mo[i]), f"momentum differs, matrix {i} step {step}"
            # the applied update  X_prev * decay - X_new  is adjusted_lr * NS(U): NS bar 2e-2
            decay = (1 - torch.tensor(lr) * torch.tensor(wd)).item()
            upd_ref = prev[i].double() * decay - Xo[i].double()
            upd_got = prev[i].double() * decay - p.detach().cpu().double()
            if dtype == torch.float32:
                assert rel_fro(upd_got, upd_ref) <= 2e-2
            # weights themselves: the NS bar scaled by how large the update is next to the weights
            # (+ one bf16 ulp of rounding noise for bf16 weights)
            bound = 2e-2 * (upd_ref.norm() / Xo[i].double().norm()).item()
            assert rel_fro(p.detach(), Xo[i]) <= bound + (4e-3 if dtype == torch.bfloat16 else 1e-6)
        # keep the two trajectories from drifting apart through the (chaotic at 1e-2) bf16 NS noise
        for i, p in enumerate(params):
            p.data.copy_(Xo[i])
    assert all(g["step"] == 3 for g in opt.param_groups)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_muon_shapes_off_the_alignment_grid(dev, dtype):
    """Dimensions that are not multiples of 8 (a flattened 3x3 convolution over 3 channels, odd square and tall
    matrices) are stepped on zero-padded copies: momentum bit exact, update within the NS bar, as for any shape."""
    from dion_amd import Muon
    from oracle import muon_step as O

    shapes = [(64, 27), (27, 64), (77, 77), (301, 100), (100, 301), (301, 100)]
    X0, gen = _make(shapes, dtype, seed=5)
    Xo = [x.clone() for x in X0]
    Mo = [torch.zeros_like(x) for x in X0]
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    lr, mu, wd = 0.02, 0.95, 0.01
    opt = Muon(params, lr=lr, mu=mu, weight_decay=wd, nesterov=True)
    for step in range(2):
        G = _grads(shapes, gen, dtype)
        for p, g in zip(params, G):
            p.grad = g.to(dev)
        prev = [x.clone() for x in Xo]
        O.muon_step(Xo, G, Mo, lr=lr, mu=mu, weight_decay=wd, epsilon=1e-8, nesterov=True)
        opt.step()
        for i, p in enumerate(params):
            assert torch.equal(opt.state[p]["momentum"].cpu(), Mo[i]), (i, step)
            decay = (1 - torch.tensor(lr) * torch.tensor(wd)).item()
            upd_ref = prev[i].double() * decay - Xo[i].double()
            if dtype == torch.float32:
                assert rel_fro(prev[i].double() * decay - p.detach().cpu().double(), upd_ref) <= 2e-2, (i, step)
            bound = 2e-2 * (upd_ref.norm() / Xo[i].double().norm()).item()
            assert rel_fro(p.detach(), Xo[i]) <= bound + (4e-3 if dtype == torch.bfloat16 else 1e-6), (i, step)
            p.data.copy_(Xo[i])


def test_muon_bf16_single_step_bits(dev):
    """With bf16 weights the update is a few ulps per element; on one step from identical state at
    least 85% of the weights must be bit-identical to the oracle's (the ~1e-2 NS noise flips some roundings)
    and none may differ by more than one ulp of the largest weight."""
    from dion_amd import Muon
    from oracle import muon_step as O

    shapes = [(768, 768), (3072, 768), (768, 3072)]
    X0, gen = _make(shapes, torch.bfloat16, seed=7)
    G = _grads(shapes, gen, torch.bfloat16)
    Xo = [x.clone() for x in X0]
    Mo = [torch.zeros_like(x) for x in X0]
    O.muon_step(Xo, G, Mo, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True)
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    for p, g in zip(params, G):
        p.grad = g.to(dev)
    Muon(params, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True).step()
    for p, xo in zip(params, Xo):
        same = (p.detach().cpu() == xo).float().mean().item()
        assert same > 0.85, same
        assert (p.detach().cpu().float() - xo.float()).abs().max().item() <= 2 ** -7 * xo.float().abs().max().item()


@pytest.mark.parametrize("adjust", ["spectral_norm", "rms_norm", "keller_muon", None])
def test_muon_adjust_lr_modes_and_groups(dev, adjust):
    from dion_amd import Muon
    from oracle import muon_step as O

    shapes = [(256, 512), (512, 256)]
    X0, gen = _make(shapes, torch.float32, seed=3)
    G = _grads(shapes, gen, torch.float32)
    Xo = [x.clone() for x in X0]
    Mo = [torch.zeros_like(x) for x in X0]
    O.muon_step(Xo, G, Mo, lr=0.01, mu=0.9, weight_decay=0.0, nesterov=False, adjust=adjust)
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    bias = torch.nn.Parameter(torch.zeros(64, device=dev))
    emb = torch.nn.Parameter(torch.randn(100, 32, device=dev))
    opt = Muon(
        [dict(params=params), dict(params=[bias], algorithm="adamw", lr=1e-3), dict(params=[emb], algorithm="lion")],
        lr=0.01, mu=0.9, weight_decay=0.0, adjust_lr=adjust,
    )
    for p, g in zip(params, G):
        p.grad = g.to(dev)
    bias.grad = torch.ones_like(bias)
    emb.grad = torch.randn_like(emb)
    e0 = emb.detach().clone()
    opt.step()
    for x0, p, xo in zip(X0, params, Xo):
        upd_ref = x0.double() - xo.double()
        upd_got = x0.double() - p.detach().cpu().double()
        assert rel_fro(upd_got, upd_ref) <= 2e-2
    # AdamW first step moves by -lr * sign(g) (bias-corrected), Lion by -lr * sign
    assert torch.allclose(bias.detach(), torch.full_like(bias, -1e-3), rtol=1e-4, atol=1e-7)
    assert torch.allclose(emb.detach(), e0 - 0.01 * torch.sign(emb.grad), atol=1e-6)
    assert set(opt.state[bias]) == {"momentum", "variance"} and set(opt.state[emb]) == {"momentum"}


def test_muon_3d_batch_flatten_and_missing_grad(dev):
    from dion_amd import Muon
    from oracle import muon_step as O

    torch.manual_seed(5)
    W = torch.randn(3, 128, 256) * 0.02       # batch of three matrices
    C = torch.randn(64, 8, 4, 4) * 0.02       # conv weight, flattened to 64 x 128
    Gw, Gc = torch.randn_like(W) * 1e-3, torch.randn_like(C) * 1e-3
    pw, pc = torch.nn.Parameter(W.clone().to(dev)), torch.nn.Parameter(C.clone().to(dev))
    unused = torch.nn.Parameter(torch.randn(128, 128, device=dev))
    opt = Muon([dict(params=[pw, unused]), dict(params=[pc], flatten=True)], lr=0.01, weight_decay=0.0)
    pw.grad, pc.grad = Gw.to(dev), Gc.to(dev)
    u0 = unused.detach().clone()
    opt.step()
    Xo, Mo = [W.clone()], [torch.zeros_like(W)]
    O.muon_step(Xo, [Gw], Mo, lr=0.01, mu=0.95, weight_decay=0.0)
    assert rel_fro(W.double() - pw.detach().cpu().double(), W.double() - Xo[0].double()) <= 2e-2
    Xc, Mc = [C.clone()], [torch.zeros_like(C)]
    O.muon_step(Xc, [Gc], Mc, lr=0.01, mu=0.95, weight_decay=0.0, flatten=True)
    assert rel_fro(C.double() - pc.detach().cpu().double(), C.double() - Xc[0].double()) <= 2e-2
    assert torch.equal(unused.detach(), u0) and unused not in opt.state


def test_muon_custom_newton_schulz_hook(dev):
    from dion_amd import Muon

    calls = []

    def hook(X, epsilon):
        calls.append((X.dtype, tuple(X.shape), float(epsilon)))
        return X  # identity "orthogonalisation"

    p = torch.nn.Parameter(torch.ones(64, 32, device=dev))
    p.grad = torch.full_like(p, 0.5)
    Muon([p], lr=0.1, mu=0.0, weight_decay=0.0, adjust_lr=None, newton_schulz_func=hook).step()
    assert calls and calls[0][0] == torch.bfloat16 and calls[0][1] == (64, 32)
    assert abs(calls[0][2] - 1e-8) < 1e-12
    assert torch.allclose(p.detach(), torch.full_like(p, 1 - 0.1 * 0.5), atol=1e-3)  # U * lr rounds in bf16


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_muon_hook_path_matches_oracle(dev, dtype):
    """The plug-in hook path (stand-alone momentum pass and weight update around a user function) against the
    oracle's step with the same function: a deterministic element-wise stand-in for the orthogonalisation, so every
    tensor must match bit for bit -- 2-D, a batch of matrices, a flattened conv weight and a column count off the
    8-grid."""
    from dion_amd import Muon
    from oracle import muon_step as O

    def stand_in(X, epsilon):
        assert X.dtype == torch.bfloat16 and X.ndim in (2, 3)
        return (X.float() * 3.0).bfloat16() - (X.float() * X.float()).bfloat16()

    shapes = [(64, 96), (64, 96), (3, 32, 40), (16, 4, 3, 3), (40, 27)]
    gen = torch.Generator().manual_seed(21)
    X0 = [(torch.randn(s, generator=gen) * 0.02).to(dtype) for s in shapes]
    Xo, Mo = [x.clone() for x in X0], [torch.zeros_like(x) for x in X0]
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    groups = [dict(params=[params[0], params[1], params[2], params[4]]), dict(params=[params[3]], flatten=True)]
    opt = Muon(groups, lr=0.02, mu=0.9, weight_decay=0.01, nesterov=True, newton_schulz_func=stand_in)
    for step in range(3):
        G = [(torch.randn(s, generator=gen) * 1e-1).to(dtype) for s in shapes]
        for p, g in zip(params, G):
            p.grad = g.to(dev)
        for i in range(len(shapes)):
            O.muon_step([Xo[i]], [G[i]], [Mo[i]], lr=0.02, mu=0.9, weight_decay=0.01, nesterov=True,
                        flatten=(i == 3), ns_func=stand_in)
        opt.step()
        for i, p in enumerate(params):
            assert torch.equal(opt.state[p]["momentum"].cpu(), Mo[i]), (step, i)
            assert torch.equal(p.detach().cpu(), Xo[i]), (step, i)


def test_newton_schulz_accepts_16_byte_aligned_views(dev):
    """A contiguous view such as `grad[1]` of a 3 x 136 x 200 tensor starts 16-byte, not 256-byte, aligned: it goes
    through the C entry point as it is and gives what a fresh copy of the same matrix gives."""
    from dion_amd import _lib
    from dion_amd.newton_schulz import NS_SCHEDULE_COEFFS, flat_coeffs

    lib = _lib.load()
    torch.manual_seed(3)
    big = torch.randn(3, 136, 200, device=dev).bfloat16()
    view = big[1]
    assert view.data_ptr() % 256 != 0 and view.data_ptr() % 16 == 0
    outs = []
    for src in (view, view.clone()):
        out_all = torch.empty(2, 136, 200, dtype=torch.bfloat16, device=dev)
        out = out_all[1] if src is view else out_all[0]
        ws = torch.empty(lib.dion_amd_ns_workspace_bytes(1, 136, 200, _lib.BF16), dtype=torch.uint8, device=dev)
        rc = lib.dion_amd_newton_schulz(src.data_ptr(), _lib.BF16, 136 * 200, 200, out.data_ptr(), 136 * 200, 200,
                                        1, 136, 200, flat_coeffs(NS_SCHEDULE_COEFFS), 5, 1e-7, _lib.BF16, 1,
                                        ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev))
        assert rc == 0, rc
        outs.append(out.clone())
    assert torch.equal(outs[0], outs[1])
    # 8 bytes off: refused, nothing launched
    flat = torch.zeros(136 * 200 + 8, dtype=torch.bfloat16, device=dev)
    rc = lib.dion_amd_newton_schulz(flat.data_ptr() + 8, _lib.BF16, 136 * 200, 200, out.data_ptr(), 136 * 200, 200,
                                    1, 136, 200, flat_coeffs(NS_SCHEDULE_COEFFS), 5, 1e-7, _lib.BF16, 1,
                                    ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev))
    assert rc == -2


def test_muon_step_buckets_equals_per_bucket_calls(dev):
    """The multi-bucket entry (grouped launches, more buckets than one grouped launch takes, a bucket
    of more matrices than one staging launch takes, shapes that are not multiples of the tile) gives
    per matrix what dion_amd_muon_step gives for each bucket on its own."""
    import ctypes

    from dion_amd import _lib
    from dion_amd.newton_schulz import NS_SCHEDULE_COEFFS, flat_coeffs

    lib = _lib.load()
    gen = torch.Generator().manual_seed(11)
    specs = [((256, 256), 5), ((128, 512), 3), ((512, 128), 3), ((40, 24), 2), ((16, 32), 70), ((8, 24), 1)]
    coeffs = flat_coeffs(NS_SCHEDULE_COEFFS)
    steps = len(NS_SCHEDULE_COEFFS)

    def fresh():
        g2 = torch.Generator().manual_seed(12)
        out = []
        for shape, nb in specs:
            X = [(torch.randn(shape, generator=g2) * 0.02).bfloat16().to(dev) for _ in range(nb)]
            G = [(torch.randn(shape, generator=g2) * 1e-3).bfloat16().to(dev) for _ in range(nb)]
            M = [(torch.randn(shape, generator=g2) * 1e-3).bfloat16().to(dev) for _ in range(nb)]
            out.append((X, G, M))
        return out

    single = fresh()
    for (shape, nb), (X, G, M) in zip(specs, single):
        m, n = shape
        ws = torch.empty(lib.dion_amd_muon_workspace_bytes(nb, m, n), dtype=torch.uint8, device=dev)
        rc = lib.dion_amd_muon_step(_lib.ptr_array(X), _lib.ptr_array(G), _lib.ptr_array(M), nb, m, n, _lib.BF16,
                                    _lib.BF16, 0.95, 1, 0.9998, 0.02 * (m / n) ** 0.5, coeffs, steps, 1e-8, 1,
                                    ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev))
        _lib.check(rc, "dion_amd_muon_step")

    multi = fresh()
    arr = (_lib.MuonBucket * len(specs))()
    keep = []
    for b, (shape, nb), (X, G, M) in zip(arr, specs, multi):
        ptrs = [_lib.ptr_array(t) for t in (X, G, M)]
        keep.append(ptrs)
        b.X, b.G, b.M = (ctypes.cast(a, ctypes.POINTER(ctypes.c_void_p)) for a in ptrs)
        b.batch, b.m, b.n = nb, shape[0], shape[1]
        b.decay, b.adjusted_lr = 0.9998, 0.02 * (shape[0] / shape[1]) ** 0.5
    need = lib.dion_amd_muon_buckets_workspace_bytes(arr, len(specs))
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    # one byte short: refused before anything is launched
    assert lib.dion_amd_muon_step_buckets(arr, len(specs), _lib.BF16, _lib.BF16, 0.95, 1, coeffs, steps, 1e-8, 1,
                                          ws.data_ptr(), need - 1, _lib.stream_ptr(dev)) == -3
    rc = lib.dion_amd_muon_step_buckets(arr, len(specs), _lib.BF16, _lib.BF16, 0.95, 1, coeffs, steps, 1e-8, 1,
                                        ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev))
    _lib.check(rc, "dion_amd_muon_step_buckets")
    torch.cuda.synchronize()
    for (shape, nb), (Xs, _, Ms), (Xm, _, Mm) in zip(specs, single, multi):
        for j in range(nb):
            assert torch.equal(Ms[j], Mm[j]), f"momentum differs: {shape} #{j}"
            # tile configuration may differ between a grouped and a single launch; accumulation order
            # per output element does not, so the weights agree to the last bit
            assert torch.equal(Xs[j], Xm[j]), f"weights differ: {shape} #{j}"


def test_muon_hook_returning_fp32_keeps_its_precision(dev):
    """A `newton_schulz_func` that returns fp32 (e.g. for fp32 weights): the reference scales and subtracts the update in
    the dtype the hook returned (dion/muon.py:569-573); the stand-alone weight update takes that dtype as it is --
    bit for bit against the oracle, which a bf16 rounding of the hook's result would not survive."""
    from dion_amd import Muon
    from oracle import muon_step as O

    def stand_in(X, epsilon):
        return X.float() * 0.37 + X.float() * X.float()

    shapes = [(64, 96), (40, 27)]
    gen = torch.Generator().manual_seed(23)
    X0 = [torch.randn(s, generator=gen) * 0.02 for s in shapes]
    Xo, Mo = [x.clone() for x in X0], [torch.zeros_like(x) for x in X0]
    params = [torch.nn.Parameter(x.clone().to(dev)) for x in X0]
    opt = Muon(params, lr=0.02, mu=0.9, weight_decay=0.01, nesterov=True, newton_schulz_func=stand_in)
    for step in range(2):
        G = [torch.randn(s, generator=gen) * 1e-1 for s in shapes]
        for p, g in zip(params, G):
            p.grad = g.to(dev)
        for i in range(len(shapes)):
            O.muon_step([Xo[i]], [G[i]], [Mo[i]], lr=0.02, mu=0.9, weight_decay=0.01, nesterov=True, ns_func=stand_in)
        opt.step()
        for i, p in enumerate(params):
            assert torch.equal(opt.state[p]["momentum"].cpu(), Mo[i]), (step, i)
            assert torch.equal(p.detach().cpu(), Xo[i]), (step, i)
