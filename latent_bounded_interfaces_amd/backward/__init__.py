"""Backward-engine side callers of the HIP kernels (counterpart of reference backward/): every name the
reference's package exports (backward/__init__.py), plus the structured providers of this package."""
from . import autograd, base, local_vjp, pullbacks, scan, suffix_scan
from .autograd import *  # noqa: F401,F403
from .base import *  # noqa: F401,F403
from .local_vjp import *  # noqa: F401,F403
from .pullbacks import *  # noqa: F401,F403
from .scan import *  # noqa: F401,F403
from .suffix_scan import *  # noqa: F401,F403

__all__ = sorted({name for module in (autograd, base, local_vjp, pullbacks, scan, suffix_scan)
                  for name in module.__all__})
