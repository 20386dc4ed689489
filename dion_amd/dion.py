"""`Dion` optimizer whose matrix path runs on the MI355X kernels.

Signature-compatible with the reference class (dion/dion.py:75-231): same constructor
arguments, defaults, validation errors, param-group keys and `self.state` layout
(`state[p]["momentum"]`, `state[p]["Q"]`, plus `"variance"` for AdamW groups).  One GPU only:
`replicate_mesh`, `outer_shard_mesh` and `inner_shard_mesh` must be None.

Per `step()` the matrices of every "dion" group are bucketed by (shape, dtype) and each bucket
goes, as arrays of device pointers, to `dion_amd_dion_step_qr`: B = M + G, the tall-skinny MFMA
GEMMs P = B Q and R = B^T P, a CholeskyQR orthonormalisation of P on the device (an fp32 pass on the bf16 matrix
cores, an fp64 pass for the factors whose measured defect asks for it, a closed-form polishing step; no host
synchronisation), the column normalisation that yields the next Q, and error feedback and weight update as one
pass over M and X.
"""
import math
import os
from collections import defaultdict
from concurrent.futures import ThreadPoolExecutor
from concurrent.futures import wait as wait_futures
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

import torch
from torch import Tensor
from torch.optim.optimizer import Optimizer, ParamsT

from . import _lib
from .elementwise_opts import adamw_update_foreach, lion_update_foreach


@dataclass
class DionMixedPrecisionConfig:
    """dtypes of the optimizer states (reference dion/dion.py:59-72); None = the parameter's dtype."""

    momentum_dtype: Optional[torch.dtype] = None
    Q_dtype: Optional[torch.dtype] = None
    variance_dtype: Optional[torch.dtype] = None



def _enqueue_dion_step(fn, device, args):
    """One bucket's library call, made by a worker thread (ctypes releases the interpreter lock for its duration)."""
    torch.cuda.set_device(device)
    return fn(*args)


class Dion(Optimizer):
    _REFERENCE_OPTIONS = False   # True in DionReference: power_iters >= 1 and all three qr_method names
    """
    Dion (https://arxiv.org/abs/2504.05295) for a single MI355X.

    Args (identical to the reference, dion/dion.py:105-124):
        params: parameters or param-group dicts; `algorithm` in {"dion", "lion", "adamw"}.
        replicate_mesh, outer_shard_mesh, inner_shard_mesh: must be None (one GPU).
        replicate_mesh_grad_sync: accepted; irrelevant on one GPU.
        rank_fraction, rank_multiple_of: r = multiple_of * ceil(fraction * min(m, n) / multiple_of).
        lr, mu, betas, weight_decay, epsilon: as in the reference.
        power_iters: must be 1.  qr_method: must be "rcqr" (the batched reference class accepts nothing else); the
            device orthonormaliser yields the reference's factor up to column signs without drawing a sketch.
        cqr_warmup_steps: steps during which `DionReference` runs "rcqr" in place of "cqr".
        rcqr_oversample: sketch rows per rank (`DionReference` with "rcqr" draws the reference's sketches).
        mixed_precision_config: dtypes of momentum / Q / variance.
    """

    def __init__(
        self,
        params: ParamsT,
        replicate_mesh=None,
        outer_shard_mesh=None,
        inner_shard_mesh=None,
        replicate_mesh_grad_sync: bool = True,
        rank_fraction: float = 1.0,
        rank_multiple_of: int = 1,
        lr: float = 0.01,
        mu: float = 0.95,
        betas: Tuple[float, float] = (0.9, 0.95),
        weight_decay: float = 0.01,
        epsilon: float = 1e-8,
        power_iters: int = 1,
        qr_method: str = "rcqr",
        cqr_warmup_steps: int = 150,
        rcqr_oversample: float = 1.25,
        mixed_precision_config: Optional[DionMixedPrecisionConfig] = None,
    ):
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if mu < 0.0:
            raise ValueError(f"Invalid momentum factor (mu): {mu}")
        if len(betas) != 2 or betas[0] < 0.0 or betas[1] < 0.0:
            raise ValueError(f"Invalid betas: {betas}")
        if weight_decay < 0.0:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        if rank_fraction <= 0 or rank_fraction > 1:
            raise ValueError(f"Invalid rank fraction: {rank_fraction}")
        if rank_multiple_of <= 0:
            raise ValueError(f"Invalid rank multiple of: {rank_multiple_of}")
        if self._REFERENCE_OPTIONS:
            # the per-matrix reference class (dion/dion_reference.py:131-134)
            if power_iters <= 0:
                raise ValueError(f"Invalid power iterations: {power_iters}")
            if qr_method not in ("qr", "cqr", "rcqr"):
                raise ValueError(f"Unknown QR method: {qr_method}")
        else:
            if power_iters != 1:
                raise ValueError("Async Dion only supports power_iters=1")
            if qr_method != "rcqr":
                raise ValueError("Async Dion only supports qr_method='rcqr'")
        for name, mesh in (("replicate_mesh", replicate_mesh), ("outer_shard_mesh", outer_shard_mesh),
                           ("inner_shard_mesh", inner_shard_mesh)):
            if mesh is not None:
                raise NotImplementedError(
                    f"dion_amd.Dion runs on one GPU: {name} must be None (got {type(mesh).__name__})."
                )

        defaults = dict(
            rank_fraction=rank_fraction, rank_multiple_of=rank_multiple_of, lr=lr, mu=mu,
            beta1=betas[0], beta2=betas[1], weight_decay=weight_decay, epsilon=epsilon,
            oversample=rcqr_oversample, algorithm="dion", step=0,
        )
        super().__init__(params, defaults)

        self._power_iters = power_iters
        self._qr_method = qr_method
        self._cqr_warmup_steps = cqr_warmup_steps
        self._replicate_mesh = None
        self._outer_shard_mesh = None
        self._inner_shard_mesh = None
        self._replicate_mesh_grad_sync = replicate_mesh_grad_sync
        self._replicate_world_size = 1
        if mixed_precision_config is None:
            mixed_precision_config = DionMixedPrecisionConfig()
        self._mixed_precision_config = mixed_precision_config
        # Buckets are independent tasks; like the reference's AsyncRuntime(max_concurrent_tasks=3)
        # (dion/dion.py:268) up to three of them are in flight, here on HIP streams of their own
        # (default priority), each with its own workspace.  The orthonormaliser is a chain of short
        # launches that cannot fill the GPU, so buckets overlap nearly for free.
        self._max_concurrent_tasks = 3
        self._workspaces = [_lib.Workspace() for _ in range(self._max_concurrent_tasks)]
        self._streams = {}
        self._info = {}
        self._pool = None   # worker threads that enqueue the buckets of a wave side by side
        self._rng = None    # generator of the random sketches (DionReference with qr_method "rcqr")

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        dion_groups, lion_groups, adamw_groups = [], [], []
        for group in self.param_groups:
            group["step"] += 1
            algo = group["algorithm"]
            if algo == "dion":
                dion_groups.append(group)
            elif algo == "lion":
                lion_groups.append(group)
            elif algo == "adamw":
                adamw_groups.append(group)
            else:
                raise ValueError(f"Unknown algorithm: {algo}")

        for group in dion_groups:
            self._dion_group_step(group)
        for group in lion_groups:
            self._lion_group_step(group)
        for group in adamw_groups:
            self._adamw_group_step(group)
        return loss

    @torch.no_grad()
    def synchronize_for_checkpoint(self):
        """No-op on one GPU (reference dion/dion.py:273-287)."""
        return

    def cholesky_info(self) -> Dict[Tuple, Tensor]:
        """Device tensors with the orthonormaliser's per-matrix status of the last step, keyed by bucket
        (shape, dtype, gradient dtype, device):
        0 = success, k > 0 = pivot k-1 was not positive (the analogue of `torch.linalg.cholesky_ex`'s info)."""
        return dict(self._info)

    def load_state_dict(self, state_dict):
        """`Optimizer.load_state_dict` casts every floating-point state tensor to its parameter's dtype, which would
        turn an fp32 `Q` or variance of bf16 weights into bf16.  The saved dtypes are those of the
        `DionMixedPrecisionConfig` the state was created with (reference dion/dion.py:636-647, 684-688, 718), and a
        checkpoint restore in the reference's trainer loads into the existing tensors and keeps them
        (train.py:566-571): keep them here as well."""
        super().load_state_dict(state_dict)
        saved_ids = [i for g in state_dict["param_groups"] for i in g["params"]]
        params = [p for g in self.param_groups for p in g["params"]]
        for pid, p in zip(saved_ids, params):
            for key, value in state_dict["state"].get(pid, {}).items():
                if torch.is_tensor(value) and value.is_floating_point() and self.state[p][key].dtype != value.dtype:
                    self.state[p][key] = value.detach().to(device=p.device, copy=True)

    # ------------------------------------------------------------------ state
    def _get_or_initialize_state(self, param: Tensor, group: dict) -> dict:
        state = self.state[param]
        algo = group["algorithm"]
        if not state:
            if algo == "dion":
                self._init_opt_state_dion(param, state, group["rank_fraction"], group["rank_multiple_of"])
            elif algo == "adamw":
                self._init_opt_state_adam(param, state)
            elif algo == "lion" or algo == "clion":
                self._init_opt_state_momentum(param, state)
            else:
                raise ValueError(f"Unknown algorithm: {algo}")
        return state

    def _init_opt_state_momentum(self, param: Tensor, state: Dict[str, Any]):
        state["momentum"] = torch.zeros_like(param, dtype=self._mixed_precision_config.momentum_dtype)

    def _init_opt_state_adam(self, param: Tensor, state: Dict[str, Any]):
        self._init_opt_state_momentum(param, state)
        state["variance"] = torch.zeros_like(param, dtype=self._mixed_precision_config.variance_dtype)

    def _init_opt_state_dion(self, param: Tensor, state: Dict[str, Any], rank_fraction: float, rank_multiple_of: int):
        """momentum = 0 and Q ~ N(0, 1) of shape (n, r), or (m, r) when m < n (reference dion/dion.py:649-721)."""
        if param.ndim != 2:
            raise ValueError(
                f"Expected Dion parameters to be 2D matrix, but got {param.ndim}D. "
                f"For scalar parameters, set 'algorithm' to 'lion' or 'adamw' when creating param group."
            )
        self._init_opt_state_momentum(param, state)
        m, n = param.shape
        r = rank_fraction * min(m, n)
        r = rank_multiple_of * math.ceil(r / rank_multiple_of)
        r = min(r, m, n)
        q_shape = (m, r) if m < n else (n, r)
        q_dtype = self._mixed_precision_config.Q_dtype
        if q_dtype is None:
            q_dtype = param.dtype
        state["Q"] = torch.randn(q_shape, device=param.device, dtype=q_dtype)

    # ------------------------------------------------------------------ dion
    def _dion_group_step(self, group: dict):
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        for p in params:
            if p.ndim > 2:
                raise NotImplementedError(
                    f"Tensors with more than 2 dimensions are not supported. Got {p.ndim}D tensor."
                )
        # hyper-parameters as 0-dim fp32 tensors, evaluated like reference dion/dion.py:327-331, 852, 859-870
        lr = torch.tensor(group["lr"])
        mu = torch.tensor(group["mu"])
        weight_decay = torch.tensor(group["weight_decay"])
        epsilon = torch.tensor(group["epsilon"])
        ef_alpha = -(1 - mu)
        decay = 1 - lr * weight_decay

        buckets = defaultdict(list)
        for p in params:
            buckets[(p.shape, p.dtype, p.grad.dtype, p.device)].append(p)
        lib = _lib.load()
        # optimizer state and status words are created on the caller's stream, before any fork
        for (shape, dtype, gdtype, device), plist in buckets.items():
            _lib.require_gpu(plist[0], "Dion.step")
            for p in plist:
                self._get_or_initialize_state(p, group)
            key = (shape, dtype, gdtype, device)
            info = self._info.get(key)
            if info is None or info.numel() != len(plist):
                self._info[key] = torch.zeros(len(plist), dtype=torch.int32, device=device)
        slots = min(len(buckets), self._max_concurrent_tasks)
        # A bucket's step is one library call that enqueues a few hundred launches on the bucket's stream.  With
        # several buckets the calls of a wave (one bucket per stream) are made by worker threads side by side: at a
        # low rank the step is otherwise bound by the time one thread needs to enqueue it, not by the GPU.
        threaded = (slots > 1 and not os.environ.get("DION_AMD_DION_SERIAL")
                    and not torch.cuda.is_current_stream_capturing())
        if threaded and getattr(self, "_pool", None) is None:
            self._pool = ThreadPoolExecutor(max_workers=self._max_concurrent_tasks, thread_name_prefix="dion_amd")
        forked = {}
        items = list(buckets.items())
        pending = []
        # Whatever happens while a wave is put together -- a non-contiguous tensor, an allocation that fails, a
        # library call that returns an error -- the calls already handed to worker threads are waited for (they hold
        # raw pointers into tensors of this frame) and the forked streams are joined before the exception travels on.
        try:
            for wave0 in range(0, len(items), slots):
                pending = []
                for index in range(wave0, min(wave0 + slots, len(items))):
                    (shape, dtype, gdtype, device), plist = items[index]
                    slot = index % slots
                    main = torch.cuda.current_stream(device)
                    if slots == 1:
                        stream = main
                    else:
                        pool = self._streams.setdefault(device, [])
                        while len(pool) < slots:
                            pool.append(torch.cuda.Stream(device=device))
                        stream = pool[slot]
                        if (device, slot) not in forked:
                            stream.wait_stream(main)   # gradients and earlier updates were produced on `main`
                            forked[(device, slot)] = (main, stream)
                    states = [self._get_or_initialize_state(p, group) for p in plist]
                    m, n = shape
                    Ms = [s["momentum"] for s in states]
                    Qs = [s["Q"] for s in states]
                    r = Qs[0].size(1)
                    for t in (*plist, *Ms, *Qs):
                        if not t.is_contiguous():
                            raise _lib.DionAmdError("Dion.step: parameters and optimizer states must be contiguous")
                    scaled_lr = ((m / n) ** 0.5) * lr
                    mcode = _lib.dtype_code(Ms[0].dtype)
                    info = self._info[(shape, dtype, gdtype, device)]
                    with torch.cuda.device(device), torch.cuda.stream(stream):
                        # contiguous gradient copies and the workspace belong to this stream
                        Xs = plist
                        Gs = [p.grad if p.grad.is_contiguous() else p.grad.contiguous() for p in plist]
                        crops = []
                        if m % 8 or n % 8:
                            # step zero-padded copies (exact: see _lib.zero_padded) and crop the results back
                            m, n = _lib.padded_dims(m, n)
                            Xw, Gw, Mw = (_lib.zero_padded(t, m, n) for t in (plist, Gs, Ms))
                            Qw = _lib.zero_padded(Qs, min(m, n), r)
                            crops = [(plist, Xw), (Ms, Mw), (Qs, Qw)]
                            Xs, Gs, Ms, Qs = (list(t.unbind(0)) for t in (Xw, Gw, Mw, Qw))
                        # Cholesky QR only after the warm-up, when the factors are well conditioned
                        # (reference dion/dion_reference.py:296-299)
                        qr_method = self._qr_method
                        if qr_method == "cqr" and group["step"] <= self._cqr_warmup_steps:
                            qr_method = "rcqr"
                        head = (
                            _lib.ptr_array(Xs), _lib.ptr_array(Gs), _lib.ptr_array(Ms), _lib.ptr_array(Qs),
                            len(plist), m, n, r,
                            _lib.dtype_code(dtype), _lib.dtype_code(gdtype), mcode, _lib.dtype_code(Qs[0].dtype),
                            ef_alpha.item(), decay.item(), scaled_lr.item(), epsilon.item(), 1, self._power_iters,
                        )
                        sketch = None
                        if self._REFERENCE_OPTIONS and qr_method == "rcqr" and max(m, n) > r:
                            # the per-matrix reference class preconditions with a random sketch from a generator of its own,
                            # seeded with 0 (reference dion/dion_reference.py:290-294, 764-775): one sketch per matrix and
                            # power iteration, drawn here and handed to the library
                            if self._rng is None:
                                self._rng = torch.Generator(device=device)
                                self._rng.manual_seed(0)
                            sketch = _sketch((self._power_iters * len(plist), max(m, n), r), Ms[0].dtype, device,
                                             group["oversample"], self._rng)
                            k = sketch.size(-2)
                            ws = self._workspaces[slot].get(
                                lib.dion_amd_dion_sketch_workspace_bytes(len(plist), m, n, r, mcode, k), device)
                            fn, what = lib.dion_amd_dion_step_sketch, "dion_amd_dion_step_sketch"
                            args = head + (sketch.data_ptr(), k, info.data_ptr(), ws.data_ptr(), ws.numel(),
                                           _lib.stream_ptr(device))
                        else:
                            ws = self._workspaces[slot].get(lib.dion_amd_dion_workspace_bytes(len(plist), m, n, r, mcode), device)
                            fn, what = lib.dion_amd_dion_step_qr, "dion_amd_dion_step_qr"
                            args = head + (_lib.QR_METHODS[qr_method], info.data_ptr(), ws.data_ptr(), ws.numel(),
                                           _lib.stream_ptr(device))
                        if threaded:
                            # (the tensors behind the pointers stay referenced until the call has returned)
                            pending.append((self._pool.submit(_enqueue_dion_step, fn, device, args), device, stream, crops,
                                            (Xs, Gs, Ms, Qs, ws, sketch), what))
                            continue
                        rc = fn(*args)
                        _lib.check(rc, what)
                        for dst, padded in crops:
                            _lib.crop_back(dst, padded)
                        del Xs, Gs, Ms, Qs, crops
                failure = None
                for future, device, stream, crops, keep, what in pending:
                    rc = future.result()   # every call of the wave has returned before anything is raised
                    if rc != 0 and failure is None:
                        failure = (rc, what)
                    if rc == 0 and crops:
                        with torch.cuda.device(device), torch.cuda.stream(stream):
                            for dst, padded in crops:
                                _lib.crop_back(dst, padded)
                pending = []
                if failure is not None:
                    _lib.check(*failure)
        finally:
            if pending:
                wait_futures([item[0] for item in pending])
            for main, stream in forked.values():
                main.wait_stream(stream)

    # ------------------------------------------------------------------ element-wise groups
    def _lion_group_step(self, group: dict):
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        states = [self._get_or_initialize_state(p, group) for p in params]
        lion_update_foreach(
            params, [p.grad for p in params], [s["momentum"] for s in states],
            lr=torch.tensor(group["lr"]), beta1=torch.tensor(group["beta1"]), beta2=torch.tensor(group["beta2"]),
            weight_decay=torch.tensor(group["weight_decay"]),
        )

    def _adamw_group_step(self, group: dict):
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        states = [self._get_or_initialize_state(p, group) for p in params]
        adamw_update_foreach(
            params, [p.grad for p in params], [s["momentum"] for s in states], [s["variance"] for s in states],
            lr=torch.tensor(group["lr"]), beta1=torch.tensor(group["beta1"]), beta2=torch.tensor(group["beta2"]),
            weight_decay=torch.tensor(group["weight_decay"]), step=torch.tensor(group["step"]),
            epsilon=torch.tensor(group["epsilon"]),
        )


def _sketch(p_shape, dtype, device, oversample, generator=None) -> Tensor:
    """S ~ N(0, 1/k) of shape (..., k, m) for factors of shape p_shape = (..., m, r), k = oversample * r rounded up to a
    multiple of 128 (reference dion/dion.py:1234-1261)."""
    m, r = p_shape[-2], p_shape[-1]
    k = math.ceil(oversample * r / 128.0) * 128
    std = math.sqrt(1.0 / k)
    return torch.empty((*p_shape[:-2], k, m), device=device, dtype=dtype).normal_(std=std, generator=generator)


def generate_random_sketch_matrix(P: Tensor, oversample: float = 1.25, shard_mesh_dim=None, generator=None) -> Tensor:
    """The sketch of the reference's randomised Cholesky QR (dion/dion.py:1221-1263) for a batch P of shape
    (..., m, r): S of shape (..., k, m) with k = oversample * r rounded up to a multiple of 128 and entries
    N(0, 1/k) in P's dtype, drawn from torch's generator for P's device (or from `generator`).
    `orthonormalize(P, sketch=S)` and `DionReference` (qr_method "rcqr") run the reference's sketched sequence with it;
    `Dion.step()` itself draws no sketch (its orthonormaliser preconditions with an fp32 CholeskyQR pass instead).
    One GPU: `shard_mesh_dim` must be None."""
    assert P.ndim >= 3, "P must have batch dimension"
    if shard_mesh_dim is not None:
        raise TypeError("Must use DTensor parameters for sharded random sketch.")
    return _sketch(P.shape, P.dtype, P.device, oversample, generator)


class DionReference(Dion):
    """Counterpart of the reference's per-matrix class (`dion.DionReference`, dion/dion_reference.py:64-365) on one
    GPU: the same constructor, which also takes `power_iters` >= 1 and `qr_method` in {"qr", "cqr", "rcqr"}
    (dion/dion_reference.py:131-134), and the same update (`dion_update`, dion/dion_reference.py:613-687; its
    `power_iteration`, 690-730, repeats P = orth(B Q), Q = B^T P with the unnormalised Q).

    `qr_method` selects the device orthonormaliser's first pass as the reference selects its factorisation
    (dion/dion_reference.py:733-789): "rcqr" -- CholeskyQR in fp32, and in fp64 for the matrices whose measured
    defect asks for it (the robust default, standing where the reference preconditions with a random sketch);
    "qr" -- the fp64 pass for every matrix (standing for Householder QR); "cqr" -- one fp32 CholeskyQR pass and
    nothing else, used after `cqr_warmup_steps` steps only (296-299), with the fall-back for a failed
    factorisation taken per matrix on the device (752-758).  All three return the thin-QR factor with a positive
    diagonal of R; the reference's Householder-based variants differ from it by column signs, which M and X do
    not see and Q carries consistently.  The status of the factorisations is in `cholesky_info()`.
    `state["Q"]` is updated in place rather than replaced by a new tensor."""

    _REFERENCE_OPTIONS = True
