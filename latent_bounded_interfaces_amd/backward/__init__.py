"""Backward-engine side callers of the HIP kernels (counterpart of reference backward/): every public name of
the submodules, under the names the reference's package exports them."""
from . import base, local_vjp, pullbacks, scan, suffix_scan
from .base import *  # noqa: F401,F403
from .local_vjp import *  # noqa: F401,F403
from .pullbacks import *  # noqa: F401,F403
from .scan import *  # noqa: F401,F403
from .suffix_scan import *  # noqa: F401,F403

__all__ = sorted({name for module in (base, local_vjp, pullbacks, scan, suffix_scan) for name in module.__all__})
