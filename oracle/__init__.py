"""CPU oracle for the Muon / Dion optimizer-step hot path.

TEST INFRASTRUCTURE ONLY.  Everything in this package is an eager-PyTorch CPU
restatement of the reference algorithm (microsoft/dion, `dion/muon.py`,
`dion/dion.py`, `dion/dion_reference.py`, `dion/muon_reference.py`), written to
be the checker the HIP path is compared with.  Only the test-suite, the smoke
check and the benchmark's CPU-baseline leg may import it; the product package
never does and has no CPU fallback.

How each function is pinned (none of them is "parity unpinned"):

* `newton_schulz.ns5`, `ns5_keller`     -- fp64 evaluation against the SVD closed
  form (`ns5_closed_form`: the iteration acts on singular values only), transpose
  equivariance, power-of-two scale invariance, and the committed golden vectors
  under `tests/golden/` produced by the reference implementation itself.
* `muon_step.muon_pre/muon_post`        -- brute-force scalar loops with explicit
  round-to-nearest-even bf16 emulation (`bf16.round_bf16`) on small inputs.
* `dion_step.dion_update`               -- projection identities (P P^T B),
  full-rank closed form M_new = mu * B, sketch-seed and sign invariance of M and X,
  unit column norms of Q, the all-zero special case, fp64 Householder truth, and
  golden vectors from the reference under `tests/golden/`.
"""
