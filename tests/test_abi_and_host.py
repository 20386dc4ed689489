"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares, and the
host-side mirror of the reference's optimizer interface validates and dispatches like the reference
(reference dion/muon.py:55-131, dion/dion.py:105-231).  No GPU compute is launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "dion_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dion_amd_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from dion_amd import _lib

    names = _declared_functions()
    assert len(names) >= 14
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/dion_amd.h but not exported"
    # and the ctypes binding covers them all
    assert set(names) == set(_lib.exported_symbols())
    lib2 = _lib.load()
    assert lib2.dion_amd_version().startswith(b"dion_amd")


def test_workspace_queries_and_argument_errors_without_gpu():
    from dion_amd import _lib

    lib = _lib.load()
    per = lib.dion_amd_ns_workspace_bytes(1, 768, 3072, _lib.BF16)
    assert per >= 2 * 768 * 3072 * 2 + 2 * 768 * 768 * 2
    assert lib.dion_amd_ns_workspace_bytes(48, 768, 768, _lib.BF16) >= 48 * 4 * 768 * 768 * 2
    assert lib.dion_amd_ns_workspace_bytes(0, 768, 768, _lib.BF16) == 0
    assert lib.dion_amd_muon_workspace_bytes(96, 4096, 14336) <= (4 << 30) + (1 << 20)  # chunked to ~4 GiB
    assert lib.dion_amd_dion_workspace_bytes(24, 3072, 768, 192, _lib.BF16) > 0
    # argument validation happens before anything is launched
    coeffs = _lib.float_array([1.0, 1.0, 1.0])
    assert lib.dion_amd_newton_schulz(None, 0, 0, 8, None, 0, 8, 1, 8, 8, coeffs, 1, 1e-7, 0, 1, None, 0, None) == -1
    assert lib.dion_amd_profile_read(99, None, None, None) == -1
    with pytest.raises(_lib.DionAmdError):
        _lib.check(-2, "x")
    with pytest.raises(_lib.DionAmdError):
        _lib.dtype_code(torch.float16)


def test_gemm_plan_keeps_huge_operands_off_the_32_bit_offset_path():
    """The direct-to-LDS K loop addresses a tile's operand with 32-bit byte offsets: an operand whose tile spans
    4 GiB or more (a k-strided bf16 matrix of 131136 rows x 16384 columns, as in R = B^T P of a vocabulary-sized layer) must
    take the bounds-checked loop.  Host-side query, nothing is launched."""
    from dion_amd import _lib

    lib = _lib.load()
    # interior tiles, small operands: 256-wide tile on the direct path
    assert lib.dion_amd_gemm_plan(4096, 4096, 4096, 4096, 0, 4096, 0) == 257
    # A k-strided with (K - 1) * ld * 2 bytes = 131135 * 16384 * 2 >= 2^32: checked loop
    assert lib.dion_amd_gemm_plan(16384, 512, 131136, 16384, 1, 512, 1) % 2 == 0
    # just below the limit stays on the direct path
    assert lib.dion_amd_gemm_plan(16384, 512, 131008, 16384, 1, 512, 1) % 2 == 1
    # a k-contiguous operand is addressed per tile row: (tile rows - 1) x pitch
    assert lib.dion_amd_gemm_plan(4096, 4096, 4096, 1 << 25, 0, 4096, 0) % 2 == 0
    assert lib.dion_amd_gemm_plan(4096, 4096, 4096, 1 << 20, 0, 4096, 0) % 2 == 1
    # ragged sizes never take it
    assert lib.dion_amd_gemm_plan(200, 136, 72, 72, 0, 72, 0) % 2 == 0
    assert lib.dion_amd_gemm_plan(0, 8, 8, 8, 0, 8, 0) == -1


def test_no_cpu_fallback():
    from dion_amd import Dion, Muon, _lib, zeropower_via_newtonschulz5

    with pytest.raises(_lib.DionAmdError):
        zeropower_via_newtonschulz5(torch.randn(16, 32))
    p = torch.nn.Parameter(torch.randn(16, 8))
    p.grad = torch.randn(16, 8)
    with pytest.raises(_lib.DionAmdError):
        Muon([p]).step()
    with pytest.raises(_lib.DionAmdError):
        Dion([p]).step()


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "dion_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"


def test_muon_constructor_contract():
    from dion_amd import Muon, _lib

    p = [torch.nn.Parameter(torch.randn(8, 8))]
    opt = Muon(p)
    assert opt.defaults == dict(lr=0.01, mu=0.95, beta1=0.9, beta2=0.95, weight_decay=0.01, algorithm="muon", step=0,
                                epsilon=1e-8, nesterov=False, flatten=False, adjust_lr="spectral_norm")
    for kw in (dict(lr=-1.0), dict(mu=-0.1), dict(betas=(0.9,)), dict(betas=(-0.1, 0.9)), dict(adjust_lr="bogus")):
        with pytest.raises(ValueError):
            Muon(p, **kw)
    with pytest.raises(TypeError):
        Muon(p, newton_schulz_func=3)
    with pytest.raises(NotImplementedError):
        Muon(p, distributed_mesh=object())
    Muon(p, use_triton=True, adjust_lr=None)  # accepted
    bad = Muon([dict(params=p, algorithm="sgd")])
    with pytest.raises(ValueError, match="Unknown algorithm"):
        bad.step()
    assert bad.param_groups[0]["step"] == 1
    vec = Muon([torch.nn.Parameter(torch.randn(8))])
    vec.param_groups[0]["params"][0].grad = torch.zeros(8)
    with pytest.raises(AssertionError):
        vec.step()
    # parameters without gradients are skipped; element-wise groups need GPU tensors like the rest
    w = torch.nn.Parameter(torch.randn(4, 4))
    e = torch.nn.Parameter(torch.ones(5))
    e.grad = torch.ones(5)
    opt = Muon([dict(params=[w]), dict(params=[e], algorithm="adamw", lr=0.1, weight_decay=0.0)])
    with pytest.raises(_lib.DionAmdError):
        opt.step()
    assert w not in opt.state and set(opt.state[e]) == {"momentum", "variance"}


def test_dion_constructor_contract():
    from dion_amd import Dion, DionMixedPrecisionConfig

    p = [torch.nn.Parameter(torch.randn(8, 8))]
    opt = Dion(p)
    assert opt.defaults == dict(rank_fraction=1.0, rank_multiple_of=1, lr=0.01, mu=0.95, beta1=0.9, beta2=0.95,
                                weight_decay=0.01, epsilon=1e-8, oversample=1.25, algorithm="dion", step=0)
    for kw in (dict(lr=-1.0), dict(mu=-1.0), dict(betas=(1.0,)), dict(weight_decay=-1.0), dict(rank_fraction=0.0),
               dict(rank_fraction=1.5), dict(rank_multiple_of=0), dict(power_iters=2), dict(qr_method="qr")):
        with pytest.raises(ValueError):
            Dion(p, **kw)
    for kw in ("replicate_mesh", "outer_shard_mesh", "inner_shard_mesh"):
        with pytest.raises(NotImplementedError):
            Dion(p, **{kw: object()})
    cfg = DionMixedPrecisionConfig(momentum_dtype=torch.bfloat16, Q_dtype=torch.float32, variance_dtype=torch.bfloat16)
    opt = Dion([dict(params=p, rank_fraction=0.5, rank_multiple_of=3)], mixed_precision_config=cfg)
    st = opt._get_or_initialize_state(p[0], opt.param_groups[0])
    assert st["momentum"].dtype == torch.bfloat16 and st["Q"].dtype == torch.float32
    assert st["Q"].shape == (8, 6)                       # 3 * ceil(0.5 * 8 / 3) = 6
    wide = torch.nn.Parameter(torch.randn(4, 16))
    st = opt._get_or_initialize_state(wide, dict(algorithm="dion", rank_fraction=1.0, rank_multiple_of=1))
    assert st["Q"].shape == (4, 4)                       # m < n: Q is (m, r)
    with pytest.raises(ValueError):
        opt._get_or_initialize_state(torch.nn.Parameter(torch.randn(4)), dict(algorithm="dion", rank_fraction=1.0,
                                                                               rank_multiple_of=1))
    a = torch.nn.Parameter(torch.ones(3))
    st = opt._get_or_initialize_state(a, dict(algorithm="adamw"))
    assert st["variance"].dtype == torch.bfloat16
    opt.synchronize_for_checkpoint()                     # no-op on one GPU
    bad = Dion([dict(params=p, algorithm="nope")])
    with pytest.raises(ValueError, match="Unknown algorithm"):
        bad.step()




def test_reference_import_paths_exist():
    """The reference exposes the orthogonalisation under three module paths (dion/muon.py:620,
    dion/newton_schulz_triton.py:305-337, dion/muon_reference.py:10); the same names import here."""
    import inspect

    from dion_amd import muon, muon_reference, newton_schulz_triton as nst
    assert list(inspect.signature(muon.zeropower_via_newtonschulz5).parameters) == ["G", "epsilon"]
    assert list(inspect.signature(nst.zeropower_via_newtonschulz5).parameters) == ["G", "epsilon"]
    assert list(inspect.signature(nst.newton_schulz_triton).parameters) == ["G", "epsilon"]
    assert list(inspect.signature(muon_reference.zeropower_via_newtonschulz5).parameters) == ["G", "steps", "eps"]
    assert callable(nst.ns_line_1) and callable(nst.ns_line_2)


def test_dion_reference_constructor_contract():
    """The per-matrix reference class's extra options (reference dion/dion_reference.py:131-134)."""
    from dion_amd import Dion, DionReference

    p = [torch.nn.Parameter(torch.randn(8, 8))]
    for method in ("qr", "cqr", "rcqr"):
        opt = DionReference(p, qr_method=method, power_iters=3, cqr_warmup_steps=7)
        assert isinstance(opt, Dion) and opt._power_iters == 3 and opt._qr_method == method
        assert opt._cqr_warmup_steps == 7 and opt.defaults == Dion(p).defaults
    with pytest.raises(ValueError, match="Invalid power iterations"):
        DionReference(p, power_iters=0)
    with pytest.raises(ValueError, match="Unknown QR method"):
        DionReference(p, qr_method="svd")
    with pytest.raises(NotImplementedError):
        DionReference(p, replicate_mesh=object())


def test_zero_padding_helpers():
    """Shapes off the 8-element grid are stepped on zero-padded copies: the padded dimensions keep which side is
    the longer one (it decides the transposes), and the copies round-trip."""
    from dion_amd import _lib

    assert _lib.padded_dims(768, 3072) == (768, 3072)
    assert _lib.padded_dims(100, 60) == (104, 64)
    assert _lib.padded_dims(60, 100) == (64, 104)
    assert _lib.padded_dims(77, 77) == (80, 80)
    assert _lib.padded_dims(100, 101) == (104, 112)      # m < n must stay m < n
    assert _lib.padded_dims(101, 100) == (112, 104)      # m > n must stay m > n
    assert _lib.padded_dims(1, 7) == (8, 16)
    mats = [torch.arange(6.0).reshape(2, 3), -torch.arange(6.0).reshape(2, 3)]
    big = _lib.zero_padded(mats, 8, 8)
    assert big.shape == (2, 8, 8) and torch.equal(big[1, :2, :3], mats[1]) and big[:, 2:].abs().sum() == 0
    assert big[:, :, 3:].abs().sum() == 0
    big[0, :2, :3] += 1
    out = [torch.zeros(2, 3), torch.zeros(2, 3)]
    _lib.crop_back(out, big)
    assert torch.equal(out[0], mats[0] + 1) and torch.equal(out[1], mats[1])


def test_generate_random_sketch_matrix_shape_and_scale():
    """reference dion/dion.py:1221-1263: (..., k, m) with k = oversample * r rounded up to a multiple of 128, N(0, 1/k)."""
    from dion_amd.dion import generate_random_sketch_matrix

    torch.manual_seed(0)
    S = generate_random_sketch_matrix(torch.zeros(3, 1000, 200), oversample=1.25)
    assert S.shape == (3, 256, 1000) and S.dtype == torch.float32
    assert abs(S.std().item() - (1.0 / 256) ** 0.5) <= 2e-4 and abs(S.mean().item()) <= 2e-4
    S = generate_random_sketch_matrix(torch.zeros(1, 64, 512, dtype=torch.bfloat16), oversample=1.0)
    assert S.shape == (1, 512, 64) and S.dtype == torch.bfloat16
    with pytest.raises(AssertionError):
        generate_random_sketch_matrix(torch.zeros(10, 4))
    with pytest.raises(TypeError):
        generate_random_sketch_matrix(torch.zeros(1, 10, 4), shard_mesh_dim=0)
