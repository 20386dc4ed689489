#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ by running the reference implementation.

Run ONLY in a container where the reference tree is mounted (default /root/reference):

    TORCHDYNAMO_DISABLE=1 python tests/golden/make_golden.py [--reference /root/reference]

The reference's functions are imported from its own tree and called on small seeded inputs;
only the input / output arrays are stored (float32 arrays hold bf16 values exactly).  Nothing
of the reference's source is copied.  TORCHDYNAMO_DISABLE=1 makes the `@torch.compile`-decorated
reference functions run eagerly, which is the op-by-op sequence the oracle restates.
"""
import argparse
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def f32(t):
    return t.detach().to(torch.float32).cpu().clone().numpy()  # clone: later in-place updates must not leak in


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reference", default="/root/reference")
    args = ap.parse_args()
    os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")
    sys.path.insert(0, args.reference)
    import dion.muon as ref_muon
    import dion.muon_reference as ref_muon_reference
    import dion.dion as ref_dion

    out = {}

    # ---- Newton-Schulz, schedule coefficients (dion/muon.py:620-647)
    for name, shape, scale in (("wide", (64, 128), 1.0), ("tall", (128, 64), 1e-3), ("square", (96, 96), 1.0)):
        g = torch.Generator().manual_seed(100)
        G = torch.randn(shape, generator=g) * scale
        out[f"ns_{name}_in"] = f32(G)
        out[f"ns_{name}_out"] = f32(ref_muon.zeropower_via_newtonschulz5(G, epsilon=1e-7))
    g = torch.Generator().manual_seed(101)
    Gb = torch.randn((3, 32, 64), generator=g)
    out["ns_batch_in"] = f32(Gb)
    out["ns_batch_out"] = f32(ref_muon.zeropower_via_newtonschulz5(Gb, epsilon=1e-7))

    # ---- Newton-Schulz, Keller coefficients (dion/muon_reference.py:10-27)
    for name, shape in (("wide", (64, 128)), ("tall", (128, 64))):
        g = torch.Generator().manual_seed(102)
        G = torch.randn(shape, generator=g)
        out[f"keller_{name}_in"] = f32(G)
        out[f"keller_{name}_out"] = f32(ref_muon_reference.zeropower_via_newtonschulz5(G, steps=5, eps=1e-7))

    # ---- Muon momentum / update passes (dion/muon.py:525-573)
    for dt_name, dt in (("bf16", torch.bfloat16), ("f32", torch.float32)):
        g = torch.Generator().manual_seed(103)
        G = (torch.randn((32, 64), generator=g) * 1e-3).to(dt)
        M = (torch.randn((32, 64), generator=g) * 1e-3).to(dt)
        X = (torch.randn((32, 64), generator=g) * 0.02).to(dt)
        out[f"muon_{dt_name}_G"], out[f"muon_{dt_name}_M0"], out[f"muon_{dt_name}_X0"] = f32(G), f32(M), f32(X)
        for nest in (False, True):
            Mi = M.clone()
            U = ref_muon.muon_update_pre_orthogonalize([G], [Mi], torch.tensor(0.95), nest)
            tag = f"muon_{dt_name}_{'nesterov' if nest else 'plain'}"
            out[tag + "_M1"], out[tag + "_U"] = f32(Mi), f32(U[0])
        Xi = X.clone()
        Uo = (torch.randn((32, 64), generator=g) * 0.1).to(torch.bfloat16)
        lr, wd = torch.tensor(0.02), torch.tensor(0.01)
        ref_muon.muon_update_post_orthogonalize([Xi], [Uo], base_lr=lr,
                                                adjusted_lr=ref_muon.adjust_lr_spectral_norm(lr, X.shape), weight_decay=wd)
        out[f"muon_{dt_name}_Uo"], out[f"muon_{dt_name}_X1"] = f32(Uo), f32(Xi)

    # ---- Dion single-GPU update (dion/dion.py:742-875), two steps, tall and wide, fp32 and bf16 momentum
    for dt_name, mdt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        for name, shape, r in (("tall", (96, 64), 16), ("wide", (64, 96), 16), ("square", (64, 64), 64)):
            g = torch.Generator().manual_seed(104)
            xdt = torch.float32 if mdt == torch.float32 else torch.bfloat16
            X = (torch.randn(shape, generator=g) * 0.02).to(xdt)
            M = torch.zeros(shape, dtype=mdt)
            qrows = min(shape)
            Q = torch.randn((qrows, r), generator=g)
            tag = f"dion_{dt_name}_{name}"
            out[tag + "_X0"], out[tag + "_Q0"] = f32(X), f32(Q)
            cfg = ref_dion._DionParamConfig()
            cfg.is_transposed = shape[0] < shape[1]
            torch.manual_seed(7)  # the sketch matrix comes from the global generator
            for step in range(2):
                G = (torch.randn(shape, generator=g) * 1e-3).to(xdt)
                out[f"{tag}_G{step}"] = f32(G)
                gen = ref_dion.dion_update_ddp(
                    X=[X], G=[G], M=[M], Q=[Q], lr=torch.tensor(0.01), mu=torch.tensor(0.95),
                    weight_decay=torch.tensor(0.01), epsilon=torch.tensor(1e-8), param_config=cfg,
                    replicate_mesh=None, replicate_mesh_grad_sync=True, oversample=torch.tensor(1.25))
                for _ in gen:
                    pass
                out[f"{tag}_X{step + 1}"], out[f"{tag}_M{step + 1}"], out[f"{tag}_Q{step + 1}"] = f32(X), f32(M), f32(Q)

    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
