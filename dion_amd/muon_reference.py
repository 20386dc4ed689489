"""Import-path twin of reference dion/muon_reference.py for the orthogonalisation function only
(`zeropower_via_newtonschulz5(G, steps=5, eps=1e-7)`, lines 10-27: fixed Keller coefficients, 2-D input)."""
from .newton_schulz import zeropower_via_newtonschulz5_keller as zeropower_via_newtonschulz5

__all__ = ["zeropower_via_newtonschulz5"]
