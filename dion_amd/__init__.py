"""MI355X-native Muon / Dion optimizer step (drop-in for the `dion` package's single-GPU path)."""
from .dion import Dion, DionMixedPrecisionConfig, DionReference  # noqa: F401
from .muon import Muon  # noqa: F401
from .newton_schulz import zeropower_via_newtonschulz5  # noqa: F401
