"""Lion / AdamW updates for the non-matrix parameter groups (embeddings, lm_head, norms, biases).

Same signatures as the reference's `lion_update_foreach` / `adamw_update_foreach`
(dion/scalar_opts.py:152-187, 89-149); the work is one fused HIP pass per call
(`dion_amd_lion_step`, `dion_amd_adamw_step`) that reproduces the rounding of each of the
reference's tensor ops.  GPU tensors only: there is no CPU or PyTorch fallback.
"""
import ctypes
from collections import defaultdict
from typing import List

import torch
from torch import Tensor

from . import _lib


def _buckets(what, *lists):
    """Indices of the tensors grouped by (device, dtypes): one library call per bucket."""
    out = defaultdict(list)
    for i, ts in enumerate(zip(*lists)):
        for t in ts:
            _lib.require_gpu(t, what)
            if not t.is_contiguous():
                raise _lib.DionAmdError(f"{what}: parameters, gradients and optimizer states must be contiguous")
        if any(t.shape != ts[0].shape for t in ts):
            raise _lib.DionAmdError(f"{what}: shapes of a parameter and its gradient / states differ")
        if ts[0].numel() == 0:
            continue
        out[(ts[0].device, *(t.dtype for t in ts))].append(i)
    return out


def _scalar(t) -> float:
    """fp32 value of a hyper-parameter expression (the reference evaluates them on 0-dim fp32 tensors)."""
    return float(torch.as_tensor(t, dtype=torch.float32))


def lion_update_foreach(X: List[Tensor], G: List[Tensor], M: List[Tensor],
                        lr: Tensor, beta1: Tensor, beta2: Tensor, weight_decay: Tensor):
    """reference dion/scalar_opts.py:152-187."""
    assert len(X) == len(G) == len(M)
    lib = _lib.load()
    lr, beta1, beta2, weight_decay = (torch.as_tensor(t, dtype=torch.float32) for t in (lr, beta1, beta2, weight_decay))
    for (device, xd, gd, md), idx in _buckets("lion_update_foreach", X, G, M).items():
        n = (ctypes.c_longlong * len(idx))(*[X[i].numel() for i in idx])
        with torch.cuda.device(device):
            rc = lib.dion_amd_lion_step(
                _lib.ptr_array([X[i] for i in idx]), _lib.ptr_array([G[i] for i in idx]),
                _lib.ptr_array([M[i] for i in idx]), n, len(idx),
                _lib.dtype_code(xd), _lib.dtype_code(gd), _lib.dtype_code(md),
                _scalar(lr), _scalar(1 - beta1), _scalar(1 - beta2), _scalar(1 - lr * weight_decay),
                _lib.stream_ptr(device))
        _lib.check(rc, "dion_amd_lion_step")


def adamw_update_foreach(X: List[Tensor], G: List[Tensor], M: List[Tensor], V: List[Tensor],
                         lr: Tensor, beta1: Tensor, beta2: Tensor, weight_decay: Tensor, step, epsilon):
    """reference dion/scalar_opts.py:89-149."""
    assert len(X) == len(G) == len(M) == len(V)
    lib = _lib.load()
    lr, beta1, beta2, weight_decay = (torch.as_tensor(t, dtype=torch.float32) for t in (lr, beta1, beta2, weight_decay))
    bias_correction1 = 1 - beta1**step
    bias_correction2 = 1 - beta2**step
    for (device, xd, gd, md, vd), idx in _buckets("adamw_update_foreach", X, G, M, V).items():
        n = (ctypes.c_longlong * len(idx))(*[X[i].numel() for i in idx])
        with torch.cuda.device(device):
            rc = lib.dion_amd_adamw_step(
                _lib.ptr_array([X[i] for i in idx]), _lib.ptr_array([G[i] for i in idx]),
                _lib.ptr_array([M[i] for i in idx]), _lib.ptr_array([V[i] for i in idx]), n, len(idx),
                _lib.dtype_code(xd), _lib.dtype_code(gd), _lib.dtype_code(md), _lib.dtype_code(vd),
                _scalar(lr / bias_correction1), _scalar(1 - beta1), _scalar(1 - beta2),
                _scalar(1 - lr * weight_decay), _scalar(bias_correction2.sqrt()), float(epsilon),
                _lib.stream_ptr(device))
        _lib.check(rc, "dion_amd_adamw_step")
