"""`Muon.step()` and `Dion.step()` captured in a HIP graph and replayed: the library enqueues kernels only (no memset,
no memcpy, no host synchronisation; reference steps dion/muon.py:133-171 and dion/dion.py:234-270 are ordinary stream
work too), so a captured step must replay to the same bits as the eager step -- on every replay, with eager work and
synchronisations between the replays."""
import pytest
import torch

pytestmark = pytest.mark.gpu

BF = torch.bfloat16
SHAPES = [(768, 768)] * 4 + [(3072, 768)] * 2 + [(768, 3072)] * 2 + [(256, 512)] * 3


def _make(kind, dev, X):
    from dion_amd import Dion, DionMixedPrecisionConfig, Muon

    params = [torch.nn.Parameter(x.clone()) for x in X]
    for p in params:
        p.grad = torch.zeros_like(p)
    if kind == "muon":
        opt = Muon(params, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True)
    else:
        torch.manual_seed(9)
        opt = Dion(params, rank_fraction=0.25, lr=0.01, mu=0.95, weight_decay=0.01,
                   mixed_precision_config=DionMixedPrecisionConfig(momentum_dtype=BF, Q_dtype=torch.float32))
    return opt, params


@pytest.mark.parametrize("kind", ["muon", "dion"])
def test_step_captured_in_a_graph_replays_bit_identically(dev, kind):
    gen = torch.Generator(device=dev).manual_seed(41)
    X = [(torch.randn(s, generator=gen, device=dev) * 0.02).to(BF) for s in SHAPES]
    grads = [[(torch.randn(s, generator=gen, device=dev) * 1e-3).to(BF) for s in SHAPES] for _ in range(5)]
    eager, pe = _make(kind, dev, X)
    graphed, pg = _make(kind, dev, X)
    if kind == "dion":
        for a, b in zip(pe, pg):
            graphed.state[b]  # (states are created lazily: take the eager optimizer's Q below)
    # two eager warm-up steps on both (workspaces, streams and states exist before the capture)
    for step in range(2):
        for opt, params in ((eager, pe), (graphed, pg)):
            for p, g in zip(params, grads[step]):
                p.grad.copy_(g)
            opt.step()
        if kind == "dion" and step == 0:
            for a, b in zip(pe, pg):
                graphed.state[b]["Q"].copy_(eager.state[a]["Q"])
                graphed.state[b]["momentum"].copy_(eager.state[a]["momentum"])
                b.data.copy_(a.data)
    torch.cuda.synchronize()
    for a, b in zip(pe, pg):
        assert torch.equal(a.detach(), b.detach())
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    snapshot = None
    if kind == "dion":   # the capture itself runs no kernel: the state must not move
        snapshot = [graphed.state[p]["momentum"].clone() for p in pg]
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            graphed.step()
    torch.cuda.synchronize()
    if snapshot is not None:
        for p, m in zip(pg, snapshot):
            assert torch.equal(graphed.state[p]["momentum"], m)
    for step in range(2, 5):
        for p, g in zip(pe, grads[step]):
            p.grad.copy_(g)
        eager.step()
        for p, g in zip(pg, grads[step]):
            p.grad.copy_(g)
        graph.replay()
        # eager work of the program's own between the replays
        junk = torch.randn(1 << 20, device=dev).sum()
        torch.cuda.synchronize()
        assert torch.isfinite(junk)
        for i, (a, b) in enumerate(zip(pe, pg)):
            assert torch.equal(a.detach(), b.detach()), f"{kind}: weights differ after replay {step - 1}, matrix {i}"
            assert torch.equal(eager.state[a]["momentum"], graphed.state[b]["momentum"]), f"{kind}: momentum, matrix {i}"
            if kind == "dion":
                assert torch.equal(eager.state[a]["Q"], graphed.state[b]["Q"]), f"{kind}: Q, matrix {i}"
