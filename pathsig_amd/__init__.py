"""pathsig for AMD MI355X: signature and log-signature operators on hand-written HIP kernels.

Same public surface as the reference package (`src/pathsig/__init__.py:5-8`):
`Signature`, `LogSignature`, `projections`.
"""
from ._load import ensure_loaded as _ensure_loaded

_ensure_loaded()

from .modules import LogSignature, Signature  # noqa: E402
from .projections import projections  # noqa: E402

__all__ = ["Signature", "LogSignature", "projections"]
