"""Oracle for the Lion / AdamW updates of the non-matrix parameter groups (test infrastructure only).

Eager PyTorch multi-tensor ops in the op sequence of the reference's `adamw_update_foreach`
(dion/scalar_opts.py:89-149) and `lion_update_foreach` (dion/scalar_opts.py:152-187): every
tensor op rounds its result to the dtype of the tensor that holds it.  Hyper-parameters are
0-dim tensors as the callers wrap them (dion/muon.py:275-353, dion/dion.py:387-473).
Pinned by the textbook closed forms in fp64 and by an explicit fp32-with-bf16-rounding
evaluation of the same sequence (tests/test_oracle_math.py).
"""
from typing import List

import torch
from torch import Tensor


def adamw_update_foreach(X: List[Tensor], G: List[Tensor], M: List[Tensor], V: List[Tensor],
                         lr: Tensor, beta1: Tensor, beta2: Tensor, weight_decay: Tensor, step, epsilon):
    """reference dion/scalar_opts.py:89-149."""
    n = len(X)
    assert n == len(G) == len(M) == len(V)
    m_dtype, v_dtype = M[0].dtype, V[0].dtype
    G = [g.to(dtype=m_dtype) for g in G]
    torch._foreach_lerp_(M, G, [1 - beta1] * n)
    G_square = torch._foreach_mul(G, G)
    G_square = [g.to(dtype=v_dtype) for g in G_square]
    torch._foreach_lerp_(V, G_square, [1 - beta2] * n)
    bias_correction1 = 1 - beta1**step
    bias_correction2 = 1 - beta2**step
    bias_correction2_sqrt = bias_correction2.sqrt()
    denom = torch._foreach_sqrt(V)
    torch._foreach_div_(denom, bias_correction2_sqrt)
    torch._foreach_add_(denom, [epsilon] * n)
    adj_lr = lr / bias_correction1
    torch._foreach_mul_(X, 1 - lr * weight_decay)
    M_div = torch._foreach_div(M, denom)
    torch._foreach_mul_(M_div, adj_lr)
    torch._foreach_sub_(X, M_div)


def lion_update_foreach(X: List[Tensor], G: List[Tensor], M: List[Tensor],
                        lr: Tensor, beta1: Tensor, beta2: Tensor, weight_decay: Tensor):
    """reference dion/scalar_opts.py:152-187."""
    n = len(X)
    assert n == len(G) == len(M)
    dtype = M[0].dtype
    G = [g.to(dtype=dtype) for g in G]
    U = torch._foreach_lerp(M, G, [1 - beta1] * n)
    torch._foreach_sign_(U)
    torch._foreach_lerp_(M, G, [1 - beta2] * n)
    torch._foreach_mul_(X, 1 - lr * weight_decay)
    torch._foreach_mul_(U, lr)
    torch._foreach_sub_(X, U)
