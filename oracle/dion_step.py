"""Oracle for one single-GPU Dion step (test infrastructure only).

Follows reference dion/dion.py `dion_update_ddp` with `replicate_mesh=None` (742-875):
`torch._foreach_add_` (794), `tensor_list_to_batch` (1200-1218), `P = M_batch @ Q_batch` (801),
`orthogonalize` (1267-1308, with `generate_random_sketch_matrix` 1221-1263),
`R = M_batch.mT @ P` (839), `fix_all_zero_or_nan` (1416-1444), `foreach_baddbmm_` (1494-1530),
`column_normalize` (1460-1491), `update_Q_matrix_` (1533-1561); state initialisation
`_init_opt_state_dion` (649-721).  `orthogonalize_variant` adds the per-matrix variants of
reference dion/dion_reference.py:733-789 ("qr", "cqr", "rcqr"), and `dion_update_reference` the per-matrix
update of the same file (613-687) with its `power_iteration` (690-730): any number of power iterations,
any of the three methods.  Pinned in tests/test_oracle_math.py: with one iteration it equals `dion_update`,
with more its M and X equal the closed form B - (1 - mu) Pk Pk^T B, Pk = thin-QR factor of B (B^T B)^(k-1) Q,
evaluated in fp64.

Everything is eager PyTorch on the CPU, one matrix per batch as on one GPU; dtypes follow
the tensors exactly as in the reference (bf16 momentum => bf16 P, R, Q_new and products).
"""
import math

import torch


def rank_of(m, n, rank_fraction, rank_multiple_of=1):
    """reference dion/dion.py:672-676"""
    r = rank_fraction * min(m, n)
    r = rank_multiple_of * math.ceil(r / rank_multiple_of)
    return int(min(r, m, n))


def sketch_matrix(P, oversample, generator=None):
    """reference dion/dion.py:1234-1261: S ~ N(0, 1/k), k = 128 ceil(oversample r / 128), in P's dtype."""
    m, r = P.size(-2), P.size(-1)
    k = math.ceil(oversample * r / 128.0) * 128
    std = math.sqrt(1.0 / k)
    return torch.empty((*P.shape[:-2], k, m), dtype=P.dtype).normal_(std=std, generator=generator)


def orthogonalize(P, oversample=1.25, generator=None, sketch=None):
    """reference dion/dion.py:1274-1308 (batched input, fp32 internally, result in P's dtype).  `sketch`: the random
    sketch S to use instead of drawing one (what the reference obtains from generate_random_sketch_matrix, 1287)."""
    assert P.ndim >= 3
    original_dtype = P.dtype
    if P.size(-2) <= P.size(-1):
        Pl, _ = torch.linalg.qr(P.to(dtype=torch.float32))
    else:
        S = sketch if sketch is not None else sketch_matrix(P, oversample, generator)
        SP = S @ P
        _, R = torch.linalg.qr(SP.to(dtype=torch.float32), mode="r")
        Pl = torch.linalg.solve_triangular(R, P.to(dtype=torch.float32), upper=True, left=False)
        PP = Pl.mT @ Pl
        R, _ = torch.linalg.cholesky_ex(PP, upper=True)
        Pl = torch.linalg.solve_triangular(R, Pl, upper=True, left=False)
    return Pl.to(original_dtype).contiguous()


def orthogonalize_variant(P, qr_method="rcqr", oversample=1.25, generator=None):
    """reference dion/dion_reference.py:733-789 (single 2-D matrix)."""
    assert qr_method in ("qr", "cqr", "rcqr")
    m, n = P.shape
    original_dtype = P.dtype
    if qr_method == "cqr":
        P32 = P.to(dtype=torch.float32)
        R, info = torch.linalg.cholesky_ex(P32.T @ P32, upper=True)
        if info == 0:
            Q = torch.linalg.solve_triangular(R, P32, upper=True, left=False)
        else:
            qr_method = "rcqr"
    if qr_method == "qr" or (qr_method == "rcqr" and m <= n):
        Q, _ = torch.linalg.qr(P.to(dtype=torch.float32))
    if qr_method == "rcqr" and m > n:
        Q = orthogonalize(P.unsqueeze(0), oversample, generator)[0].to(torch.float32)
    return Q.to(dtype=original_dtype)


def fix_all_zero_or_nan(P, R, Q_init, B):
    """reference dion/dion.py:1437-1444"""
    is_all_zero = (B == 0).all(dim=(-2, -1), keepdim=True)
    not_all_zero = ~is_all_zero
    P = P.nan_to_num() * not_all_zero
    R = R.nan_to_num() * not_all_zero + Q_init * is_all_zero
    return P, R


def column_normalize(X, epsilon):
    """reference dion/dion.py:1477-1491"""
    original_dtype = X.dtype
    Xl = X.to(dtype=torch.float32)
    ss = Xl.square().sum(dim=-2, keepdim=True)
    Xl = Xl / (torch.sqrt(ss) + epsilon)
    return Xl.to(original_dtype)


def baddbmm_(X, A, B, alpha, beta, transpose):
    """reference dion/dion.py:1513-1530 (one matrix per batch)."""
    update = (A @ B.mT) if not transpose else (B @ A.mT)
    update = update.unbind(dim=0)
    update = torch._foreach_mul(update, alpha)
    torch._foreach_mul_(X, beta)
    torch._foreach_add_(X, update)


def dion_update(X, G, M, Q, lr, mu, weight_decay, epsilon=1e-8, oversample=1.25, generator=None, orth=None):
    """One Dion step on a single matrix (tensors modified in place: X, M, Q).

    `orth` optionally replaces the orthonormaliser (callable on the batched P) -- used by the
    tests to show that M and X do not depend on the sketch or on column signs.
    Returns (P, R) of the step for inspection.
    """
    lr = torch.tensor(lr) if not isinstance(lr, torch.Tensor) else lr
    mu = torch.tensor(mu) if not isinstance(mu, torch.Tensor) else mu
    weight_decay = torch.tensor(weight_decay) if not isinstance(weight_decay, torch.Tensor) else weight_decay
    epsilon = torch.tensor(epsilon) if not isinstance(epsilon, torch.Tensor) else epsilon
    transposed = X.size(0) < X.size(1)                       # dion.py:531-535
    torch._foreach_add_([M], [G])                            # dion.py:794
    M_batch = torch.stack([M.mT if transposed else M])       # dion.py:1210-1213
    Q_batch = torch.stack([Q]).to(M_batch.dtype)             # dion.py:1216
    P = M_batch @ Q_batch                                    # dion.py:801
    P = (orth or (lambda p: orthogonalize(p, oversample, generator)))(P)   # dion.py:822
    R = M_batch.mT @ P                                       # dion.py:839
    P, R = fix_all_zero_or_nan(P, R, Q_batch, M_batch)       # dion.py:847
    baddbmm_([M], P, R, alpha=-(1 - mu), beta=1.0, transpose=transposed)   # dion.py:851-853
    Q_new = column_normalize(R, epsilon)                     # dion.py:856
    scaled_lr = ((X.size(0) / X.size(1)) ** 0.5) * lr        # dion.py:859-861
    baddbmm_([X], P, Q_new, alpha=-scaled_lr, beta=1 - lr * weight_decay, transpose=transposed)  # dion.py:865-872
    Q.copy_(Q_new[0].to(Q.dtype))                            # dion.py:875, 1559-1561
    return P[0], R[0]


def dion_step(X, G, M, Q, lr, mu, weight_decay, epsilon=1e-8, oversample=1.25, generator=None, orth=None):
    """One step for every matrix of the lists (in place)."""
    for x, g, m, q in zip(X, G, M, Q):
        dion_update(x, g, m, q, lr, mu, weight_decay, epsilon, oversample, generator, orth)


def dion_update_reference(X, G, M, Q, lr, mu, weight_decay, epsilon=1e-8, power_iters=1, qr_method="rcqr",
                          oversample=1.25, generator=None):
    """reference dion/dion_reference.py:613-687 with power_iteration (690-730), one matrix, no meshes.
    X and M are modified in place; returns the new Q (the reference class stores it in state["Q"], 319-325)."""
    lr = torch.tensor(lr) if not isinstance(lr, torch.Tensor) else lr
    mu = torch.tensor(mu) if not isinstance(mu, torch.Tensor) else mu
    weight_decay = torch.tensor(weight_decay) if not isinstance(weight_decay, torch.Tensor) else weight_decay
    transpose = X.size(0) < X.size(1)                         # dion_reference.py:396-420 (is_transposed)
    Q_init_dtype = Q.dtype
    Q = Q.to(M.dtype)                                         # 636-637
    M.add_(G)                                                 # 640
    B = M.T if transpose else M                               # 645
    Qi = Q
    for _ in range(power_iters):                              # 712-728
        P = B @ Qi
        P = orthogonalize_variant(P, qr_method, oversample, generator)
        Qi = B.T @ P
    R = Qi
    P, R = fix_all_zero_or_nan(P, R, Q, M)                    # 656
    if not transpose:                                         # 660-663
        M.add_(P @ R.T, alpha=-(1 - mu))
    else:
        M.add_(R @ P.T, alpha=-(1 - mu))
    R = R.to(dtype=torch.float32)                             # 668-670
    Qn = (R / (R.norm(dim=0, keepdim=True) + epsilon)).to(P.dtype)
    X.mul_(1 - lr * weight_decay)                             # 673
    scaled_lr = ((X.size(0) / X.size(1)) ** 0.5) * lr         # 676-678
    if not transpose:                                         # 682-685
        X.add_(P @ Qn.T, alpha=-scaled_lr)
    else:
        X.add_(Qn @ P.T, alpha=-scaled_lr)
    return Qn.to(Q_init_dtype)                                # 687
