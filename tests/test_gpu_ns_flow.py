"""The persistent Newton-Schulz kernel (all iterations of many small matrices in one launch; reference
dion/muon.py:620-647 iterated per matrix) against the product-by-product launches it replaces: the tiles run the
same code in the same order of k, so every result must be the same bits -- with the kernel's own cache handling
(a matrix's tiles stay behind one L2) and with an L2 write-back after every tile."""
import pytest
import torch

pytestmark = pytest.mark.gpu

BF = torch.bfloat16
GPT_SMALL_LAYER = [(768, 768)] * 4 + [(3072, 768), (768, 3072)]


@pytest.fixture
def flow_option():
    from dion_amd import _lib

    yield lambda mode: _lib.set_option("ns_flow", mode)
    _lib.set_option("ns_flow", -1)
    _lib.set_option("ns_flow_fail", 0)


def _muon_run(dev, shapes, steps, seed=1):
    from dion_amd import Muon

    gen = torch.Generator(device=dev).manual_seed(seed)
    X = [(torch.randn(s, generator=gen, device=dev) * 0.02).to(BF) for s in shapes]
    params = [torch.nn.Parameter(x.clone()) for x in X]
    opt = Muon(params, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True, adjust_lr="spectral_norm")
    for _ in range(steps):
        for p in params:
            p.grad = (torch.randn(p.shape, generator=gen, device=dev) * 1e-3).to(BF)
        opt.step()
    torch.cuda.synchronize()
    return [p.detach().clone() for p in params], [opt.state[p]["momentum"].clone() for p in params]


@pytest.mark.parametrize("shapes", [
    GPT_SMALL_LAYER * 12,                                   # 48 / 12 / 12: three groups in one launch
    [(512, 256)] * 3 + [(256, 256)] * 5,                    # fewer matrices than queues in the first group
    [(1024, 2048)] * 9 + [(256, 1280)] * 17,                # counts that do not divide by eight
])
def test_muon_step_persistent_kernel_equals_product_launches(dev, flow_option, shapes):
    runs = {}
    for mode in (0, 1, 2):
        flow_option(mode)
        runs[mode] = _muon_run(dev, shapes, 2)
    for mode in (1, 2):
        for i, (a, b) in enumerate(zip(runs[0][0], runs[mode][0])):
            assert torch.isfinite(b).all(), f"mode {mode}: non-finite weights, matrix {i}"
            assert torch.equal(a, b), f"mode {mode}: weights differ, matrix {i} {tuple(a.shape)}"
        for i, (a, b) in enumerate(zip(runs[0][1], runs[mode][1])):
            assert torch.equal(a, b), f"mode {mode}: momentum differs, matrix {i}"


@pytest.mark.parametrize("batch,m,n,steps", [(24, 768, 3072, 5), (5, 256, 512, 3), (40, 512, 512, 1), (16, 1024, 768, 6)])
def test_newton_schulz_persistent_kernel_equals_product_launches(dev, flow_option, batch, m, n, steps):
    from dion_amd.newton_schulz import newton_schulz

    torch.manual_seed(3)
    G = torch.randn(batch, m, n, device=dev).to(BF)
    coeffs = [(3.4445, -4.7750, 2.0315)] * steps
    flow_option(0)
    ref = newton_schulz(G, coeffs=coeffs)
    for mode in (1, 2):
        flow_option(mode)
        got = newton_schulz(G, coeffs=coeffs)
        torch.cuda.synchronize()
        assert torch.equal(ref, got), f"mode {mode}"


def test_a_persistent_launch_that_gave_up_poisons_the_result(dev, flow_option):
    """The status word of a launch that gave up (here: set by the host before the launch, the kernel's waits then
    end at once) turns every result into NaN instead of leaving half-iterated values behind."""
    from dion_amd import _lib
    from dion_amd.newton_schulz import newton_schulz

    torch.manual_seed(4)
    G = torch.randn(16, 512, 768, device=dev).to(BF)
    flow_option(1)
    _lib.set_option("ns_flow_fail", 1)
    out = newton_schulz(G)
    torch.cuda.synchronize()
    assert torch.isnan(out).all()
    _lib.set_option("ns_flow_fail", 0)
    out = newton_schulz(G)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
