"""State-dict round trip of the optimizers (reference dion/dion.py:636-647 state keys, train.py:495-507, 566-571
checkpoint use): a run that is saved, rebuilt from the saved state and resumed must continue like one that was never
interrupted, for the mixed-precision state variants of `DionMixedPrecisionConfig` as well."""
import copy
import io

import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPES = [(256, 128), (128, 256), (128, 128), (128, 128)]


def _make_params(dev, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    mats = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(dtype).to(dev)) for s in SHAPES]
    emb = torch.nn.Parameter((torch.randn(300, 64, generator=gen) * 0.02).to(dtype).to(dev))
    head = torch.nn.Parameter((torch.randn(300, 64, generator=gen) * 0.02).to(dtype).to(dev))
    norm = torch.nn.Parameter(torch.ones(64, dtype=dtype, device=dev))
    return mats, emb, head, norm


def _grads(params, step, dev):
    gen = torch.Generator().manual_seed(1000 + step)
    for p in params:
        p.grad = (torch.randn(p.shape, generator=gen) * 1e-2).to(p.dtype).to(dev)


def _groups(mats, emb, head, norm, algo):
    return [dict(params=mats, algorithm=algo), dict(params=[emb, norm], algorithm="lion", lr=1e-3),
            dict(params=[head], algorithm="adamw", lr=1e-3, weight_decay=0.0)]


def _through_file(sd):
    """What a checkpoint does to a state dict: serialise, read back on the CPU."""
    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    return torch.load(buf, map_location="cpu", weights_only=True)


def _run(make_opt, dev, dtype, steps_before, steps_after):
    # uninterrupted
    P = _make_params(dev, dtype, 0)
    flat = [*P[0], *P[1:]]
    torch.manual_seed(7)   # Dion draws its initial Q from the global generator at the first step
    opt = make_opt(P)
    for s in range(steps_before + steps_after):
        _grads(flat, s, dev)
        opt.step()
    # interrupted after `steps_before`
    P1 = _make_params(dev, dtype, 0)
    flat1 = [*P1[0], *P1[1:]]
    torch.manual_seed(7)
    opt1 = make_opt(P1)
    for s in range(steps_before):
        _grads(flat1, s, dev)
        opt1.step()
    sd = _through_file(copy.deepcopy(opt1.state_dict()))
    weights = [p.detach().cpu().clone() for p in flat1]
    P2 = _make_params(dev, dtype, 1)                      # different init: everything must come from the checkpoint
    flat2 = [*P2[0], *P2[1:]]
    for p, w in zip(flat2, weights):
        p.data.copy_(w)
    opt2 = make_opt(P2)
    opt2.load_state_dict(sd)
    for g, g1 in zip(opt2.param_groups, opt1.param_groups):
        assert g["step"] == g1["step"] == steps_before and g["algorithm"] == g1["algorithm"]
    for p2, p1 in zip(flat2, flat1):
        assert set(opt2.state[p2]) == set(opt1.state[p1])
        for k, v in opt1.state[p1].items():
            assert opt2.state[p2][k].dtype == v.dtype and opt2.state[p2][k].device == v.device
            assert torch.equal(opt2.state[p2][k], v)
    for s in range(steps_before, steps_before + steps_after):
        _grads(flat2, s, dev)
        opt2.step()
    return flat, opt, flat2, opt2


def test_muon_resume_is_bit_identical(dev):
    from dion_amd import Muon

    make = lambda P: Muon(_groups(*P, "muon"), lr=0.02, mu=0.95, nesterov=True, weight_decay=0.01)  # noqa: E731
    flat, opt, flat2, opt2 = _run(make, dev, torch.bfloat16, 3, 2)
    for p, p2 in zip(flat, flat2):
        assert torch.equal(p.detach(), p2.detach())
        for k in opt.state[p]:
            assert torch.equal(opt.state[p][k], opt2.state[p2][k]), k


@pytest.mark.parametrize("variant", ["fp32", "bf16_state", "bf16_momentum_fp32_q"])
def test_dion_resume_and_mixed_precision(dev, variant):
    from dion_amd import Dion, DionMixedPrecisionConfig

    bf, f32 = torch.bfloat16, torch.float32
    dtype, cfg = {
        "fp32": (f32, None),
        "bf16_state": (bf, DionMixedPrecisionConfig(momentum_dtype=bf, Q_dtype=bf, variance_dtype=bf)),
        "bf16_momentum_fp32_q": (bf, DionMixedPrecisionConfig(momentum_dtype=bf, Q_dtype=f32, variance_dtype=f32)),
    }[variant]
    make = lambda P: Dion(_groups(*P, "dion"), rank_fraction=0.25, lr=0.01, mu=0.95, weight_decay=0.01,  # noqa: E731
                          mixed_precision_config=cfg)
    flat, opt, flat2, opt2 = _run(make, dev, dtype, 3, 2)
    st = opt.state[flat[0]]
    assert st["momentum"].dtype == (cfg.momentum_dtype if cfg else dtype)
    assert st["Q"].dtype == (cfg.Q_dtype if cfg else dtype) and st["Q"].shape == (128, 32)
    assert opt.state[flat[-2]]["variance"].dtype == (cfg.variance_dtype if cfg else dtype)   # lm_head: AdamW
    # every sum of the step has a fixed order: the resumed run is the uninterrupted one bit for bit
    for p, p2 in zip(flat, flat2):
        assert torch.equal(p.detach(), p2.detach())
        for k in opt.state[p]:
            assert torch.equal(opt.state[p][k], opt2.state[p2][k]), k
