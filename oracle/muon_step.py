"""Oracle for one single-GPU Muon step on a list of matrices (test infrastructure only).

Follows reference dion/muon.py: `muon_update_pre_orthogonalize` (525-552),
`muon_update_newton_schulz` (576-593), `adjust_lr_*` (596-617),
`muon_update_post_orthogonalize` (556-573) and the single-GPU branch of
`muon_update_batch_async` (356-391, 437-448, 461-486).  Hyper-parameters are 0-dim
fp32 CPU tensors exactly as `Muon._create_muon_tasks` wraps them (muon.py:205-208).
"""
import math

import torch

from .newton_schulz import ns5


def muon_pre(G, M, momentum, nesterov):
    """reference dion/muon.py:536-552 (lists of tensors; M modified in place)."""
    dtype = M[0].dtype
    G = [g.to(dtype=dtype) for g in G]
    torch._foreach_mul_(M, momentum)
    torch._foreach_add_(M, G)
    if nesterov:
        U = torch._foreach_mul(M, momentum)
        torch._foreach_add_(U, G)
    else:
        U = M
    return [u.to(dtype=torch.bfloat16) for u in U]


def muon_post(X, U, base_lr, adjusted_lr, weight_decay):
    """reference dion/muon.py:568-573."""
    torch._foreach_mul_(X, 1 - base_lr * weight_decay)
    U = torch._foreach_mul(U, adjusted_lr)
    torch._foreach_sub_(X, U)


def adjust_lr(lr, shape, mode):
    """reference dion/muon.py:596-617 and the dispatch at 468-477."""
    if mode is None:
        return lr
    A, B = shape[-2:]
    if mode == "spectral_norm":
        return lr * math.sqrt(A / B)
    if mode == "rms_norm":
        return lr * (0.2 * math.sqrt(max(A, B)))
    if mode == "keller_muon":
        return lr * max(1, A / B) ** 0.5
    raise ValueError(f"Unknown adjust_lr value: {mode}")


def muon_newton_schulz(X, flatten, epsilon, ns_func=ns5):
    """reference dion/muon.py:585-593."""
    original_shape = X.shape
    if flatten and X.ndim >= 3:
        X = X.flatten(start_dim=1)
    elif X.ndim >= 4:
        X = X.flatten(end_dim=-3)
    return ns_func(X, epsilon=epsilon).reshape(original_shape)


def muon_step(X, G, M, lr, mu, weight_decay, epsilon=1e-8, nesterov=False, adjust="spectral_norm",
              flatten=False, ns_func=ns5):
    """One step for every matrix of the lists X, G, M (in place), one matrix per task as on one GPU."""
    lr_t = torch.tensor(lr)
    mu_t = torch.tensor(mu)
    wd_t = torch.tensor(weight_decay)
    eps_t = torch.tensor(epsilon)
    for x, g, m in zip(X, G, M):
        U = muon_pre([g], [m], mu_t, nesterov)
        u = muon_newton_schulz(U[0], flatten, eps_t, ns_func)
        muon_post([x], [u], lr_t, adjust_lr(lr_t, x.shape, adjust), wd_t)
