"""ctypes binding of `libdion_amd.so` (the C ABI declared in `include/dion_amd.h`).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# DION_AMD_LIB names another build of the same library (kernel experiments); default: in-tree
LIB_PATH = os.environ.get("DION_AMD_LIB") or os.path.join(_HERE, "libdion_amd.so")

BF16, F32, F64 = 0, 1, 2
EPI_STORE, EPI_AXPBY = 0, 1

_DTYPE_CODE = {torch.bfloat16: BF16, torch.float32: F32, torch.float64: F64}

_ERRORS = {
    -1: "bad argument (null pointer or non-positive size)",
    -2: "alignment: dimensions/pitches must be multiples of 8 (bf16) or 4 (fp32) elements, pointers 16-byte aligned",
    -3: "workspace too small",
    -4: "unsupported dtype",
    -5: "size beyond a documented limit",
}

_c = ctypes
_vp, _i, _ll, _f, _sz = _c.c_void_p, _c.c_int, _c.c_longlong, _c.c_float, _c.c_size_t
_fp = _c.POINTER(_c.c_float)
_vpp = _c.POINTER(_c.c_void_p)



class MuonBucket(ctypes.Structure):
    """`dion_amd_muon_bucket` of include/dion_amd.h."""
    _fields_ = [("X", _vpp), ("G", _vpp), ("M", _vpp), ("batch", _i), ("m", _i), ("n", _i),
                ("decay", _f), ("adjusted_lr", _f)]


_bkp = _c.POINTER(MuonBucket)

_SIGNATURES = {
    "dion_amd_version": (_c.c_char_p, []),
    "dion_amd_ns_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "dion_amd_newton_schulz": (_i, [_vp, _i, _ll, _i, _vp, _ll, _i, _i, _i, _i, _fp, _i, _f, _i, _i, _vp, _sz, _vp]),
    "dion_amd_static_scratch_bytes": (_sz, []),
    "dion_amd_newton_schulz_static": (_i, [_vp, _i, _ll, _i, _vp, _ll, _i, _i, _i, _i, _fp, _i, _f, _i, _i, _vp]),
    "dion_amd_syrk": (_i, [_vp, _ll, _i, _vp, _ll, _i, _i, _i, _i, _i, _vp]),
    "dion_amd_sym_poly": (_i, [_vp, _ll, _i, _vp, _ll, _i, _i, _i, _f, _f, _i, _i, _vp]),
    "dion_amd_gemm": (_i, [_vp, _ll, _i, _i, _vp, _ll, _i, _i, _vp, _ll, _i, _vp, _ll, _i,
                           _i, _i, _i, _i, _i, _i, _i, _f, _f, _i, _vp]),
    "dion_amd_muon_workspace_bytes": (_sz, [_i, _i, _i]),
    "dion_amd_orthonormalize_workspace_bytes": (_sz, [_i, _i, _i]),
    "dion_amd_orthonormalize": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "dion_amd_orthonormalize_method": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "dion_amd_dion_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "dion_amd_dion_bq_fused": (_i, [_i, _i, _i, _i, _i, _i]),
    "dion_amd_dion_step": (_i, [_vpp, _vpp, _vpp, _vpp, _i, _i, _i, _i, _i, _i, _i, _i, _f, _f, _f, _f, _i, _i,
                                _vp, _vp, _sz, _vp]),
    "dion_amd_dion_step_qr": (_i, [_vpp, _vpp, _vpp, _vpp, _i, _i, _i, _i, _i, _i, _i, _i, _f, _f, _f, _f, _i, _i, _i,
                                   _vp, _vp, _sz, _vp]),
    "dion_amd_set_option": (_i, [_c.c_char_p, _i]),
    "dion_amd_orthonormalize_sketch_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "dion_amd_orthonormalize_sketch": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "dion_amd_dion_sketch_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i]),
    "dion_amd_dion_step_sketch": (_i, [_vpp, _vpp, _vpp, _vpp, _i, _i, _i, _i, _i, _i, _i, _i, _f, _f, _f, _f, _i, _i,
                                       _vp, _i, _vp, _vp, _sz, _vp]),
    "dion_amd_tile_trace_enable": (_i, [_i]),
    "dion_amd_tile_trace_read": (_i, [_vp, _i]),
    "dion_amd_ns_flow_trace_enable": (_i, [_i]),
    "dion_amd_ns_flow_trace_read": (_i, [_vp, _i, _c.POINTER(_i)]),
    "dion_amd_probe": (_i, [_i, _vp, _sz, _i, _vp, _sz, _vp, _c.POINTER(_c.c_double), _vp]),
    "dion_amd_profile_enable": (_i, [_i]),
    "dion_amd_profile_reset": (_i, []),
    "dion_amd_profile_read": (_i, [_i, _c.POINTER(_ll), _c.POINTER(_c.c_double), _c.POINTER(_c.c_double)]),
    "dion_amd_muon_step": (_i, [_vpp, _vpp, _vpp, _i, _i, _i, _i, _i, _f, _i, _f, _f, _fp, _i, _f, _i, _vp, _sz, _vp]),
    "dion_amd_lion_step": (_i, [_vpp, _vpp, _vpp, _c.POINTER(_ll), _i, _i, _i, _i, _f, _f, _f, _f, _vp]),
    "dion_amd_adamw_step": (_i, [_vpp, _vpp, _vpp, _vpp, _c.POINTER(_ll), _i, _i, _i, _i, _i,
                                 _f, _f, _f, _f, _f, _f, _vp]),
    "dion_amd_muon_pre": (_i, [_vpp, _vpp, _vpp, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "dion_amd_muon_post": (_i, [_vpp, _vpp, _i, _i, _i, _i, _i, _f, _f, _vp]),
    "dion_amd_gemm_plan": (_i, [_i, _i, _i, _i, _i, _i, _i]),
    "dion_amd_muon_buckets_workspace_bytes": (_sz, [_bkp, _i]),
    "dion_amd_muon_step_buckets": (_i, [_bkp, _i, _i, _i, _f, _i, _fp, _i, _f, _i, _vp, _sz, _vp]),
}

_lib = None


class DionAmdError(RuntimeError):
    pass


def load():
    """Load the shared library (once) and declare every prototype."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise DionAmdError(
            f"{LIB_PATH} not found: the HIP extension is not built. Run `python -m dion_amd.build` "
            "(there is no CPU or PyTorch fallback)."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def exported_symbols():
    return list(_SIGNATURES)


def check(rc, what):
    if rc == 0:
        return
    if rc < 0:
        raise DionAmdError(f"{what}: {_ERRORS.get(rc, 'error')} (code {rc})")
    raise DionAmdError(f"{what}: HIP error {rc}")


def dtype_code(dtype):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise DionAmdError(f"unsupported dtype {dtype}") from None


def require_gpu(t, what):
    if not t.is_cuda:
        raise DionAmdError(
            f"{what}: tensor is on {t.device}; the MI355X kernels need a GPU tensor (no CPU fallback)"
        )


def stream_ptr(device=None):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def float_array(values):
    arr = (ctypes.c_float * len(values))(*values)
    return arr


def ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def padded_dims(m, n):
    """(m, n) rounded up to multiples of 8 (16-byte rows for the kernels) without changing which side is the
    longer one: the orientation decides the transposes of both optimizers."""
    m8, n8 = -(-m // 8) * 8, -(-n // 8) * 8
    if m < n and m8 == n8:
        n8 += 8
    if m > n and m8 == n8:
        m8 += 8
    return m8, n8


def zero_padded(mats, rows, cols):
    """A (len(mats), rows, cols) tensor holding the 2-D tensors `mats` in its top-left corners, zero elsewhere.
    Zero rows and columns go through Newton-Schulz and through a Dion step unchanged and change nothing else,
    so a shape the kernels cannot take directly is stepped on such a copy and cropped back."""
    out = mats[0].new_zeros((len(mats), rows, cols))
    for o, t in zip(out, mats):
        o[: t.size(0), : t.size(1)].copy_(t)
    return out


def crop_back(dst, padded):
    for d, s in zip(dst, padded):
        d.copy_(s[: d.size(0), : d.size(1)])


class Workspace:
    """A grow-only byte buffer taken from PyTorch's caching allocator (stream-ordered lifetime)."""

    def __init__(self):
        self._buf = None

    def get(self, nbytes, device):
        if self._buf is None or self._buf.numel() < nbytes or self._buf.device != device:
            self._buf = None
            self._buf = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        return self._buf


QR_METHODS = {"rcqr": 0, "qr": 1, "cqr": 2}   # DION_AMD_QR_*


def set_option(name, value):
    """`dion_amd_set_option`: a run-time switch of the library (e.g. "fused_update": 1 / 0 / -1 = default)."""
    check(load().dion_amd_set_option(name.encode(), int(value)), f"dion_amd_set_option({name!r})")

PROF_KINDS = ("ns_syrk", "ns_poly", "ns_axpy", "stage", "normalize", "unstage", "gemm",
              "dion_bq", "dion_btp", "dion_ef", "dion_upd", "dion_orth", "dion_elem", "scalar_opt", "dion_ef_upd", "ns_flow")


def profile_read():
    """{kind: (launches, total_ms, total_work)} for every kind with at least one recorded launch."""
    lib = load()
    out = {}
    for k, name in enumerate(PROF_KINDS):
        n, ms, work = _ll(0), _c.c_double(0), _c.c_double(0)
        check(lib.dion_amd_profile_read(k, _c.byref(n), _c.byref(ms), _c.byref(work)), "dion_amd_profile_read")
        if n.value:
            out[name] = (n.value, ms.value, work.value)
    return out
