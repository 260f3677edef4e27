"""MI355X-native kernels for the LBI bounded-interface backward hot path.

Two device routines behind the reference's own Python contracts:

* ``hip.interface.suffix_scan_pullbacks``  - suffix scan of interface pullback matrices
* ``hip.transformer.attention_input_pullback_basis`` - attention dQ/dK/dV for P basis directions

plus the callers either side of them (``backward.suffix_scan``, ``backends.transformer_hip``).
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]
__version__ = "0.1.0"
