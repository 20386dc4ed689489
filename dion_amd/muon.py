"""`Muon` optimizer whose matrix path runs on the MI355X kernels.

Signature-compatible with the reference class (dion/muon.py:25-131): same constructor
arguments and defaults, same param-group keys, same `self.state` layout
(`state[p]["momentum"]`, plus `"variance"` for AdamW groups), same exceptions.  One GPU
only: `distributed_mesh` must be None.

Per `step()` the matrices of every "muon" group are bucketed by (shape, dtype) -- the
grouping rule of `create_param_batches` (reference dion/opt_utils.py:48-65) -- and each
bucket is handed, as arrays of device pointers, to `dion_amd_muon_step`, which runs the
fused momentum pass, the batched Newton-Schulz GEMMs and the fused weight update on the
current stream.
"""
import math
from collections import defaultdict
from typing import Callable, List, Optional, Tuple

import ctypes

import torch
from torch import Tensor
from torch.optim.optimizer import Optimizer, ParamsT

from . import _lib
from .elementwise_opts import adamw_update_foreach, lion_update_foreach
from .newton_schulz import NS_SCHEDULE_COEFFS, flat_coeffs, zeropower_via_newtonschulz5


def adjust_lr_rms_norm(lr, param_shape):
    """reference dion/muon.py:596-602"""
    A, B = param_shape[-2:]
    return lr * (0.2 * math.sqrt(max(A, B)))


def adjust_lr_spectral_norm(lr, param_shape):
    """reference dion/muon.py:605-610"""
    fan_out, fan_in = param_shape[-2:]
    return lr * math.sqrt(fan_out / fan_in)


def adjust_lr_keller_muon(lr, param_shape):
    """reference dion/muon.py:612-617"""
    fan_out, fan_in = param_shape[-2:]
    return lr * max(1, fan_out / fan_in) ** 0.5


_ADJUST = {
    "spectral_norm": adjust_lr_spectral_norm,
    "rms_norm": adjust_lr_rms_norm,
    "keller_muon": adjust_lr_keller_muon,
}


class Muon(Optimizer):
    """
    Muon for a single MI355X.

    Args (identical to the reference, dion/muon.py:55-69):
        params: parameters or param-group dicts. A group may override any default and
            selects its update rule with `algorithm` in {"muon", "lion", "adamw"}.
        distributed_mesh: must be None (one GPU).
        lr, mu, betas, weight_decay, epsilon, nesterov, adjust_lr, flatten: as in the reference.
        use_triton: accepted and ignored; the HIP kernels are always used.
        newton_schulz_func: optional custom `func(input: Tensor, epsilon) -> Tensor`; when
            given, the momentum pass and the weight update run as separate kernels around that function.
    """

    def __init__(
        self,
        params: ParamsT,
        distributed_mesh=None,
        lr: float = 0.01,
        mu: float = 0.95,
        betas: Tuple[float, float] = (0.9, 0.95),
        weight_decay: float = 0.01,
        epsilon: float = 1e-8,
        nesterov: bool = False,
        adjust_lr: Optional[str] = "spectral_norm",
        flatten: bool = False,
        use_triton: bool = False,
        newton_schulz_func: Optional[Callable] = None,
    ):
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if mu < 0.0:
            raise ValueError(f"Invalid momentum factor (mu): {mu}")
        if len(betas) != 2 or betas[0] < 0.0 or betas[1] < 0.0:
            raise ValueError(f"Invalid betas: {betas}")
        if adjust_lr not in ("spectral_norm", "rms_norm", "keller_muon", None):
            raise ValueError(
                f"Invalid adjust_lr value: {adjust_lr}. Must be 'spectral_norm', 'rms_norm', 'keller_muon', or None."
            )
        defaults = dict(
            lr=lr, mu=mu, beta1=betas[0], beta2=betas[1], weight_decay=weight_decay, algorithm="muon",
            step=0, epsilon=epsilon, nesterov=nesterov, flatten=flatten, adjust_lr=adjust_lr,
        )
        super().__init__(params, defaults)

        if distributed_mesh is not None:
            raise NotImplementedError(
                "dion_amd.Muon runs on one GPU: distributed_mesh must be None "
                f"(got {type(distributed_mesh).__name__})."
            )
        self._device_rank = 0
        self._world_size = 1
        self._process_group = None
        self._distributed_mesh = None

        if newton_schulz_func is not None:
            if not callable(newton_schulz_func):
                raise TypeError(f"newton_schulz_func must be a callable function, got {type(newton_schulz_func)}")
            self._newton_schulz_func = newton_schulz_func
            self._fused = False
        else:
            self._newton_schulz_func = zeropower_via_newtonschulz5
            self._fused = True
        self._workspace = _lib.Workspace()
        self._coeffs = flat_coeffs(NS_SCHEDULE_COEFFS)

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        muon_groups, lion_groups, adamw_groups = [], [], []
        for group in self.param_groups:
            group["step"] += 1
            algo = group["algorithm"]
            if algo == "muon":
                muon_groups.append(group)
            elif algo == "lion":
                lion_groups.append(group)
            elif algo == "adamw":
                adamw_groups.append(group)
            else:
                raise ValueError(f"Unknown algorithm: {algo}")

        for group in muon_groups:
            self._muon_group_step(group)
        for group in lion_groups:
            self._lion_group_step(group)
        for group in adamw_groups:
            self._adamw_group_step(group)
        return loss

    # ------------------------------------------------------------------ state
    def _get_or_initialize_state(self, param: Tensor, algo: str) -> dict:
        state = self.state[param]
        if not state:
            state["momentum"] = torch.zeros_like(param)
            if algo == "adamw":
                state["variance"] = torch.zeros_like(param)
        return state

    # ------------------------------------------------------------------ muon
    def _muon_group_step(self, group: dict):
        assert all(p.ndim >= 2 for p in group["params"]), "Muon optimizer only supports matrix parameters."
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        adjust = group["adjust_lr"]
        if adjust is not None and adjust not in _ADJUST:
            raise ValueError(f"Unknown adjust_lr value: {adjust}")

        # hyper-parameters as 0-dim fp32 tensors, evaluated like reference dion/muon.py:205-208
        lr = torch.tensor(group["lr"])
        mu = torch.tensor(group["mu"])
        weight_decay = torch.tensor(group["weight_decay"])
        epsilon = torch.tensor(group["epsilon"])

        buckets = defaultdict(list)
        for p in params:
            buckets[(p.shape, p.dtype, p.grad.dtype, p.device)].append(p)

        # Buckets of one (dtype, grad dtype, device) go to the library together: their Newton-Schulz
        # products are grouped launches, so small buckets share the GPU instead of queueing
        # (the reference overlaps them as async tasks, dion/muon.py:185-270).
        fused = defaultdict(list)
        crops = []
        for (shape, dtype, gdtype, device), plist in buckets.items():
            states = [self._get_or_initialize_state(p, "muon") for p in plist]
            adjusted_lr = lr if adjust is None else _ADJUST[adjust](lr, shape)
            if not self._fused:
                self._muon_bucket_unfused(plist, states, lr, adjusted_lr, mu, weight_decay, epsilon, group)
                continue
            _lib.require_gpu(plist[0], "Muon.step")
            X, G, M = self._matrix_views(plist, states, group["flatten"])
            m, n = X[0].shape
            if m % 8 or n % 8:
                # step zero-padded copies (exact: see _lib.zero_padded) and crop the results back
                m8, n8 = _lib.padded_dims(m, n)
                Xw, Gw, Mw = (_lib.zero_padded(t, m8, n8) for t in (X, G, M))
                crops.append((X, Xw))
                crops.append((M, Mw))
                X, G, M = list(Xw.unbind(0)), list(Gw.unbind(0)), list(Mw.unbind(0))
            fused[(dtype, gdtype, device)].append((X, G, M, float(adjusted_lr)))

        decay = 1 - lr * weight_decay
        for (dtype, gdtype, device), items in fused.items():
            lib = _lib.load()
            arr = (_lib.MuonBucket * len(items))()
            keep = []  # pointer arrays (and contiguous gradient copies) must outlive the call
            for b, (X, G, M, alr) in zip(arr, items):
                px, pg, pm = _lib.ptr_array(X), _lib.ptr_array(G), _lib.ptr_array(M)
                keep.append((px, pg, pm, G))
                b.X, b.G, b.M = (ctypes.cast(a, ctypes.POINTER(ctypes.c_void_p)) for a in (px, pg, pm))
                b.batch = len(X)
                b.m, b.n = X[0].shape
                b.decay = decay.item()
                b.adjusted_lr = alr
            ws = self._workspace.get(lib.dion_amd_muon_buckets_workspace_bytes(arr, len(items)), device)
            with torch.cuda.device(device):
                rc = lib.dion_amd_muon_step_buckets(
                    arr, len(items), _lib.dtype_code(dtype), _lib.dtype_code(gdtype),
                    mu.item(), int(bool(group["nesterov"])),
                    self._coeffs, len(NS_SCHEDULE_COEFFS), epsilon.item(), 1,
                    ws.data_ptr(), ws.numel(), _lib.stream_ptr(device),
                )
            _lib.check(rc, "dion_amd_muon_step_buckets")
            del keep
        for dst, padded in crops:
            _lib.crop_back(dst, padded)

    @staticmethod
    def _matrix_views(plist: List[Tensor], states: List[dict], flatten: bool):
        """Split every parameter into the 2-D matrices Newton-Schulz sees (reference dion/muon.py:585-591):
        `flatten` folds trailing dims of a >=3-D tensor into columns, otherwise leading dims are a batch."""
        X, G, M = [], [], []
        for p, st in zip(plist, states):
            mom = st["momentum"]
            if not p.is_contiguous() or not mom.is_contiguous():
                raise _lib.DionAmdError("Muon.step: parameters and momentum buffers must be contiguous")
            g = p.grad if p.grad.is_contiguous() else p.grad.contiguous()
            if p.ndim == 2:
                X.append(p); G.append(g); M.append(mom)
            elif flatten:
                X.append(p.view(p.size(0), -1)); G.append(g.view(p.size(0), -1)); M.append(mom.view(p.size(0), -1))
            else:
                r, c = p.shape[-2:]
                X.extend(p.view(-1, r, c).unbind(0)); G.extend(g.view(-1, r, c).unbind(0))
                M.extend(mom.view(-1, r, c).unbind(0))
        return X, G, M

    def _muon_bucket_unfused(self, plist, states, lr, adjusted_lr, mu, weight_decay, epsilon, group):
        """Custom `newton_schulz_func` (the reference's plug-in hook, dion/muon.py:48-49, 122-131): the momentum pass
        and the weight update run as the library's stand-alone stages (`dion_amd_muon_pre` / `dion_amd_muon_post`,
        reference dion/muon.py:536-552 and 568-573) around the user's function, which is called per parameter with
        the reference's flatten rules (585-593) and a 0-dim fp32 `epsilon` tensor."""
        lib = _lib.load()
        p0 = plist[0]
        _lib.require_gpu(p0, "Muon.step")
        device = p0.device
        cols = p0.size(-1)
        rows = p0.numel() // cols
        Ms = [st["momentum"] for st in states]
        for t in (*plist, *Ms):
            if not t.is_contiguous():
                raise _lib.DionAmdError("Muon.step: parameters and momentum buffers must be contiguous")
        X = [p.view(rows, cols) for p in plist]
        G = [(p.grad if p.grad.is_contiguous() else p.grad.contiguous()).view(rows, cols) for p in plist]
        M = [m.view(rows, cols) for m in Ms]
        crops = []
        c8 = cols
        if cols % 8:
            # the stages move 16-byte row segments: step zero-padded copies and crop the results back
            c8 = -(-cols // 8) * 8
            Xw, Gw, Mw = (_lib.zero_padded(t, rows, c8) for t in (X, G, M))
            crops = [(X, Xw), (M, Mw)]
            X, G, M = list(Xw.unbind(0)), list(Gw.unbind(0)), list(Mw.unbind(0))
        U = torch.empty((len(plist), rows, c8), dtype=torch.bfloat16, device=device)
        Us = list(U.unbind(0))
        with torch.cuda.device(device):
            rc = lib.dion_amd_muon_pre(
                _lib.ptr_array(G), _lib.ptr_array(M), _lib.ptr_array(Us), len(plist), rows, c8,
                _lib.dtype_code(G[0].dtype), _lib.dtype_code(M[0].dtype), mu.item(), int(bool(group["nesterov"])),
                _lib.stream_ptr(device))
        _lib.check(rc, "dion_amd_muon_pre")
        O = []
        for p, u in zip(plist, Us):
            u = u[:, :cols].reshape(p.shape) if c8 != cols else u.view(p.shape)
            if group["flatten"] and u.ndim >= 3:
                v = u.flatten(start_dim=1)
            elif u.ndim >= 4:
                v = u.flatten(end_dim=-3)
            else:
                v = u
            o = self._newton_schulz_func(v, epsilon=epsilon).reshape(p.shape)
            # the update is scaled and subtracted in the dtype the function returned (reference dion/muon.py:569-573):
            # bf16 and fp32 go to the library as they are, anything else as fp32
            if o.dtype not in (torch.bfloat16, torch.float32):
                o = o.to(dtype=torch.float32)
            o = o.reshape(rows, cols)
            if c8 != cols:
                o = torch.nn.functional.pad(o, (0, c8 - cols))
            o = o.contiguous()
            if o.data_ptr() % 16:   # (a contiguous view at an odd offset: the kernels move 16-byte segments)
                o = o.clone()
            O.append(o)
        o_dtypes = {o.dtype for o in O}
        if len(o_dtypes) > 1:
            O = [o.to(dtype=torch.float32) for o in O]
        alr = adjusted_lr.item() if isinstance(adjusted_lr, Tensor) else float(torch.tensor(adjusted_lr).item())
        with torch.cuda.device(device):
            rc = lib.dion_amd_muon_post(
                _lib.ptr_array(X), _lib.ptr_array(O), len(plist), rows, c8, _lib.dtype_code(X[0].dtype),
                _lib.dtype_code(O[0].dtype), (1 - lr * weight_decay).item(), alr, _lib.stream_ptr(device))
        _lib.check(rc, "dion_amd_muon_post")
        for dst, padded in crops:
            _lib.crop_back(dst, padded)

    # ------------------------------------------------------------------ element-wise groups
    def _lion_group_step(self, group: dict):
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        states = [self._get_or_initialize_state(p, "lion") for p in params]
        lion_update_foreach(
            params, [p.grad for p in params], [s["momentum"] for s in states],
            lr=torch.tensor(group["lr"]), beta1=torch.tensor(group["beta1"]), beta2=torch.tensor(group["beta2"]),
            weight_decay=torch.tensor(group["weight_decay"]),
        )

    def _adamw_group_step(self, group: dict):
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        states = [self._get_or_initialize_state(p, "adamw") for p in params]
        adamw_update_foreach(
            params, [p.grad for p in params], [s["momentum"] for s in states], [s["variance"] for s in states],
            lr=torch.tensor(group["lr"]), beta1=torch.tensor(group["beta1"]), beta2=torch.tensor(group["beta2"]),
            weight_decay=torch.tensor(group["weight_decay"]), step=torch.tensor(group["step"]),
            epsilon=torch.tensor(group["epsilon"]),
        )
